"""Pins the CPU checker's two decode loops (`ko_gemma_forward`, `ko_gemma4_forward`): the composition of the
single ops, which the op-level tests cannot see.

Three kinds of evidence, none of which reuses the loops' own code:
  * `tests/loop_restatement.py`, a float64 numpy restatement of the reference's OTHER formulation of the step
    (separate q / k / v GEMVs, rmsnorm_add -> rmsnorm -> gate, up, gelu_mul -> down, textbook softmax over the
    dequantized cache), must agree with the loops to f32 noise on logits and hidden state, every step;
  * invariants that follow from the mathematics of the layer (what zeroed projections leave, what position 0
    cannot depend on, what a scale of the residual stream does);
  * sensitivity: every norm vector and every matrix is perturbed on the restatement's side only, and the
    comparison must then fail -- so a swapped or dropped operand on the loops' side could not pass it.
"""
import copy

import numpy as np
import pytest

import oracle
from ksearch_amd import synth
from tests.gpu_util import rel_err
from tests.loop_restatement import Restatement

PLAIN = dict(n_layers=3, hidden=512, ffn=1024, n_q=4, n_kv=1, hd=128, vocab=512, max_seq=160, eps=1e-6, softcap=30.0,
             rope_theta=10000.0, attn_scale=1.0 / np.sqrt(128.0))
NORMS = ("attn_norm", "q_norm", "k_norm", "post_attn_norm", "ffn_norm", "post_ffw_norm")


def plain_weights(seed=18):
    w = synth.gemma_weights(PLAIN, seed, oracle.quantize_q4k, synth.chunked(oracle.quantize_q6k), std=0.05)
    rng = np.random.default_rng(seed + 1)
    for lw in w["layers"]:
        for name in NORMS:      # distinct vectors, so that a swap of two of them shows
            lw[name] = (1.0 + 0.2 * rng.standard_normal(lw[name].size)).astype(np.float32)
    w["output_norm"] = (1.0 + 0.2 * rng.standard_normal(PLAIN["hidden"])).astype(np.float32)
    return w


def rows_of(model, owning, pos, row_bytes):
    """The packed K / V rows a checker loop appended at `pos`: [layer][which] (None where nothing is appended)."""
    out = []
    for l, rb in enumerate(row_bytes):
        if not owning[l]:
            out.append(None)
            continue
        out.append([model.kv(l, which, (pos + 1) * rb)[pos * rb:].copy() for which in (0, 1)])
    return out


def q40_steps(a, b, n):
    """Largest difference between two packed Q4_0 rows in units of the first one's block scale."""
    if np.array_equal(a, b):
        return 0.0
    va, vb = oracle.dequant(oracle.Q40, a, n).reshape(-1, 32), oracle.dequant(oracle.Q40, b, n).reshape(-1, 32)
    d = np.abs(a.reshape(-1, 18)[:, :2].copy().view(np.float16).astype(np.float32))
    with np.errstate(divide="ignore", invalid="ignore"):
        st = np.where(d > 0, np.abs(va - vb) / d, 0.0)
    return float(st.max())


def run_against_restatement(model, rs, owning, row_bytes, n_elems, steps, first_token, logit_tol=5e-4):
    """Teacher-forced run of the checker loop over a fixed random token sequence (with tied embeddings a greedy run
    of a random model repeats its input token, every cached V row is then the same and the attention no longer
    depends on q or k); the restatement is fed the same tokens and attends over the loop's packed rows.  Returns
    the worst relative logit error seen (the caller asserts on it or expects it to be large)."""
    worst, flips = 0.0, 0
    tokens = np.random.default_rng(first_token).integers(0, model.vocab, size=steps)
    for step in range(steps):
        tok = int(tokens[step])
        nxt, logits = model.forward(tok, return_logits=True)
        rows = rows_of(model, owning, step, row_bytes)
        want, hidden, own = rs.forward(tok, rows)
        worst = max(worst, float(rel_err(logits, want).max()), float(rel_err(model.hidden(), hidden).max()))
        if worst > logit_tol:
            return worst, flips
        # the rows the restatement packs from its own float64 K / V are the loop's rows up to one code of a value
        # that sits on a rounding boundary
        for l, r in enumerate(rows):
            if r is None:
                continue
            for which in (0, 1):
                st = q40_steps(r[which], own[l][which], n_elems[l])
                assert st <= 1.0 + 1e-3, (step, l, which, st)
                flips += int((r[which] != own[l][which]).sum())
        margin = np.sort(want)[-2:]
        if margin[1] - margin[0] > 1e-3 * max(1.0, abs(margin[1])):
            assert nxt == int(np.argmax(want)), step
    return worst, flips


def make_plain(w):
    m = oracle.Gemma(PLAIN, w)
    rb = [PLAIN["n_kv"] * PLAIN["hd"] // 32 * 18] * PLAIN["n_layers"]
    return m, [True] * PLAIN["n_layers"], rb, [PLAIN["n_kv"] * PLAIN["hd"]] * PLAIN["n_layers"]


def test_plain_loop_matches_the_unfused_restatement():
    w = plain_weights()
    m, owning, rb, ne = make_plain(w)
    rs = Restatement.from_plain(PLAIN, w)
    worst, flips = run_against_restatement(m, rs, owning, rb, ne, 140, 5)      # crosses the 128-row attention switch
    assert worst <= 5e-4, worst
    assert flips <= 0.01 * 140 * sum(rb) * 2, flips
    m.close()


def tiny4(**kw):
    # softmax scale 1/8: with the checkpoints' 1.0 the scores of unit-rms q and k reach +-30, the softmax is nearly
    # one-hot and f32-vs-f64 noise in a near-tie between two rows shows up at 1e-3; the scale is a plain parameter
    cfg = dict(synth.GEMMA4_TINY, vocab=256, attn_scale=0.125)
    pattern = [1, 1, 0, 1, 1, 1, 0, 1]
    w = synth.gemma4_weights(cfg, 20, oracle.quantize_q4k, oracle.quantize_q6k, ffn=[512, 512, 1024, 512, 512, 1024, 512, 512],
                             swa_pattern=pattern, **kw)
    return cfg, w


def make_g4(cfg, w):
    m = oracle.Gemma4(cfg, w)
    n = cfg["n_layers"]
    owning = [l < n - cfg["shared_kv_layers"] for l in range(n)]
    hd = [cfg["hd_swa"] if lw["is_swa"] else cfg["hd_full"] for lw in w["layers"]]
    return m, owning, [cfg["n_kv"] * h // 32 * 18 for h in hd], [cfg["n_kv"] * h for h in hd]


@pytest.mark.parametrize("q6k", [(), ((0, "wq"), (1, "wdown"), (2, "wgate"), (3, "wv"), (6, "wo"), (7, "wup"))])
def test_gemma4_loop_matches_the_unfused_restatement(q6k):
    """Both layer kinds, a window shorter than the run, three layers reading earlier caches, per-layer embeddings,
    layer scales, two feed-forward widths, Q4_K and Q6_K tensors."""
    cfg, w = tiny4(q6k_tensors=q6k)
    m, owning, rb, ne = make_g4(cfg, w)
    rs = Restatement(cfg, w)
    assert [d["src"] for d in rs.L] == [m.kv_source(l) for l in range(cfg["n_layers"])]
    worst, _ = run_against_restatement(m, rs, owning, rb, ne, 24, 9)
    assert worst <= 5e-4, worst
    m.close()


def _perturbations_plain():
    for name in NORMS + ("wq", "wk", "wv", "wo", "wgate", "wup", "wdown"):
        yield 1, name
    yield None, "output_norm"


@pytest.mark.parametrize("layer,name", list(_perturbations_plain()))
def test_plain_comparison_sees_every_operand(layer, name):
    """The comparison above is only worth something if it fails when one operand differs: every norm vector and
    every matrix of one layer is changed on the restatement's side alone (norms: swapped with another norm vector
    of the same length or reversed; matrices: rows reversed), and the agreement must be lost within 6 steps."""
    w = plain_weights()
    w2 = copy.deepcopy(w)
    if layer is None:
        w2[name] = w2[name][::-1].copy()
    elif name in NORMS:
        same_len = [n for n in NORMS if n != name and w["layers"][layer][n].size == w["layers"][layer][name].size]
        w2["layers"][layer][name] = w["layers"][layer][same_len[0]].copy()
    else:
        rows = {"wq": 512, "wk": 128, "wv": 128, "wo": 512, "wgate": 1024, "wup": 1024, "wdown": 512}[name]
        w2["layers"][layer][name] = w["layers"][layer][name].reshape(rows, -1)[::-1].copy().reshape(-1)
    m, owning, rb, ne = make_plain(w)
    rs = Restatement.from_plain(PLAIN, w2)
    try:
        worst, _ = run_against_restatement(m, rs, owning, rb, ne, 6, 5)
    except AssertionError:
        worst = 1.0                      # the packed rows or the argmax disagreed: also a detection
    assert worst > 2e-3, (name, worst)
    m.close()


@pytest.mark.parametrize("what", ["post_norm", "layer_scale", "inp_gate", "proj", "ple_proj_norm", "ple_model_proj", "ple_embd",
                                  "window", "shared"])
def test_gemma4_comparison_sees_the_extras(what):
    cfg, w = tiny4()
    cfg2, w2 = dict(cfg), copy.deepcopy(w)
    L = w2["layers"][2]
    if what == "post_norm":
        L["post_norm"] = w["layers"][2]["post_ffw_norm"].copy()
    elif what == "layer_scale":
        L["layer_scale"] = 1.0
    elif what in ("inp_gate", "proj"):
        rows = {"inp_gate": cfg["ple_dim"], "proj": cfg["hidden"]}[what]
        L[what] = L[what].reshape(rows, -1)[::-1].copy().reshape(-1)
    elif what == "ple_proj_norm":
        w2["globals"][what] = w2["globals"][what][::-1].copy()
    elif what == "ple_model_proj":
        rows = cfg["n_layers"] * cfg["ple_dim"]
        w2["globals"][what] = w2["globals"][what].reshape(rows, -1)[::-1].copy().reshape(-1)
    elif what == "ple_embd":
        w2["globals"][what] = w2["globals"][what].reshape(cfg["vocab"], -1)[::-1].copy().reshape(-1)
    elif what == "window":
        cfg2["sliding_window"] = cfg["sliding_window"] + 1
    elif what == "shared":
        cfg2["shared_kv_layers"] = 0         # every layer would attend over its own cache
    steps = 12 if what == "window" else 6
    m, owning, rb, ne = make_g4(cfg, w)
    if what == "shared":
        # give the restatement K / V projections for the layers that have none: it will pack its own rows for them
        for l in range(cfg["n_layers"] - cfg["shared_kv_layers"], cfg["n_layers"]):
            src = w2["layers"][m.kv_source(l)]
            w2["layers"][l].update(wk=src["wk"], wv=src["wv"], dt_k=src["dt_k"], dt_v=src["dt_v"])
    rs = Restatement(cfg2, w2)
    worst = 0.0
    for step, tok in enumerate(np.random.default_rng(9).integers(0, cfg["vocab"], size=steps)):
        nxt, logits = m.forward(int(tok), return_logits=True)
        rows = rows_of(m, owning, step, rb)
        want, _, _ = rs.forward(int(tok), rows)
        worst = max(worst, float(rel_err(logits, want).max()))
    assert worst > 2e-3, (what, worst)
    m.close()


def test_zeroed_output_projections_leave_the_embedding():
    """With `wo` and `wdown` zero every residual update is rms(0)*w = 0, so the stream stays the scaled embedding
    row and the logits are the LM head of its output norm, whatever the other tensors hold."""
    w = plain_weights()
    for lw in w["layers"]:
        lw["wo"] = np.zeros_like(lw["wo"])
        lw["wdown"] = np.zeros_like(lw["wdown"])
    m = oracle.Gemma(PLAIN, w)
    h = PLAIN["hidden"]
    emb = oracle.dequant(oracle.Q6K, w["token_embd"], PLAIN["vocab"] * h).astype(np.float64).reshape(-1, h)
    for tok in (3, 77, 500):
        _, logits = m.forward(tok, return_logits=True)
        x = np.sqrt(np.float32(h)).astype(np.float64) * emb[tok]
        assert float(rel_err(m.hidden(), x).max()) <= 1e-6
        want = emb @ (x / np.sqrt(np.mean(x * x) + PLAIN["eps"]) * w["output_norm"])
        assert float(rel_err(logits, want).max()) <= 1e-4
    m.close()


def test_position_zero_does_not_depend_on_q_or_k():
    """A softmax over one row is 1: at position 0 the attention output is the dequantized V row for every head,
    so the logits cannot depend on wq, wk, q_norm or k_norm; at position 1 they do."""
    w = plain_weights()
    w2 = copy.deepcopy(w)
    for lw in w2["layers"]:
        lw["wq"], lw["wk"] = lw["wq"].reshape(512, -1)[::-1].copy().reshape(-1), lw["wk"].reshape(128, -1)[::-1].copy().reshape(-1)
        lw["q_norm"], lw["k_norm"] = lw["q_norm"][::-1].copy(), lw["k_norm"][::-1].copy()
    a, b = oracle.Gemma(PLAIN, w), oracle.Gemma(PLAIN, w2)
    _, la0 = a.forward(11, return_logits=True)
    _, lb0 = b.forward(11, return_logits=True)
    assert np.array_equal(la0, lb0)
    rb = PLAIN["hd"] // 32 * 18
    for l in range(PLAIN["n_layers"]):
        assert np.array_equal(a.kv(l, 1, rb), b.kv(l, 1, rb))              # V rows equal
        assert not np.array_equal(a.kv(l, 0, rb), b.kv(l, 0, rb))          # K rows are not
    _, la1 = a.forward(12, return_logits=True)
    _, lb1 = b.forward(12, return_logits=True)
    assert float(rel_err(la1, lb1).max()) > 1e-3
    a.close()
    b.close()


def test_row_adoption_reports_and_adopts():
    """`adopt_rows` (what the GPU tests use to keep two correct implementations on one cache): handing a loop its
    own rows changes nothing and reports no difference; rows with one code moved are reported as one step and are
    what the cache holds afterwards."""
    w = plain_weights()
    a, b = oracle.Gemma(PLAIN, w), oracle.Gemma(PLAIN, w)
    rb = PLAIN["hd"] // 32 * 18
    tok = 7
    for step in range(3):
        nxt, la = a.forward(tok, return_logits=True)
        rows = np.stack([np.stack([a.kv(l, which, (step + 1) * rb)[step * rb:] for which in (0, 1)])
                         for l in range(PLAIN["n_layers"])])
        _, lb = b.forward(tok, return_logits=True, adopt_rows=rows)
        assert np.array_equal(la, lb) and not b.row_diff_bytes.any() and not b.row_max_step.any()
        tok = nxt
    rows = rows.copy()
    _ = a.forward(tok)
    rows = np.stack([np.stack([a.kv(l, which, 4 * rb)[3 * rb:] for which in (0, 1)]) for l in range(PLAIN["n_layers"])]).copy()
    rows[1, 0, 2 + 3] ^= 0x10          # layer 1, K, block 0: high nibble of byte 3 moves by one code
    b.forward(tok, adopt_rows=rows)
    assert b.row_diff_bytes[1, 0] == 1 and abs(b.row_max_step[1, 0] - 1.0) < 1e-3
    assert np.array_equal(b.kv(1, 0, 4 * rb)[3 * rb:], rows[1, 0])
    assert b.row_diff_bytes.sum() >= 1
    a.close()
    b.close()
