"""The ops and the decode loop for the real Gemma-4 checkpoints' layer features (sliding-window and full-attention
layers, shared KV caches, per-layer embeddings, mixed Q4_K / Q6_K tensors) vs the CPU oracle."""
import numpy as np
import pytest

import oracle
from ksearch_amd import hip, synth
from ksearch_amd.hip import DType, Kind
from tests.gpu_util import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = hip.Context()
    yield c
    c.close()


@pytest.fixture(scope="module")
def eng():
    return hip.Eng()


def test_dequant_q5k_bit_exact(ctx, eng):
    n = 256 * 300
    blocks = synth.q5k_blocks(n // 256, 600, 1e-3, 1e-2)
    dst = ctx.buffer_empty_f32(n)
    eng.dequant(ctx, DType.Q5K, n, ctx.buffer_bytes(blocks), dst)
    assert np.array_equal(ctx.read_f32(dst, n), oracle.dequant(oracle.Q5K, blocks, n))


@pytest.mark.parametrize("dt,rb", [(DType.Q5K, 176), (DType.Q4K, 144), (DType.Q6K, 210), (DType.F16, 512)])
def test_copy_scale_indexed_row_gather(ctx, eng, dt, rb):
    n, rows = 1024, 37
    if dt == DType.F16:
        table = synth.normal_f32(rows * n, 601).astype(np.float16)
        raw, odt = table.view(np.uint8), oracle.F16
    else:
        gen = {DType.Q5K: synth.q5k_blocks, DType.Q4K: synth.q4k_blocks, DType.Q6K: synth.q6k_blocks}[dt]
        raw, odt = gen(rows * n // 256, 601), int(dt)
    src, out, idx = ctx.buffer_bytes(raw), ctx.buffer_empty_f32(n), ctx.buffer_f32(np.array([0], np.float32))
    for rid in (0, 17, rows - 1):
        ctx.write_buffer(idx, np.array([rid], np.float32))
        k = eng._k(ctx, Kind.COPY_SCALE_INDEXED, (n, rows), (dt,), (16.0,))
        ctx.encode_multi(k, [src, idx], [out])
        assert np.array_equal(ctx.read_f32(out, n), oracle.copy_scale_indexed(odt, raw, rid, n, 16.0)), rid


@pytest.mark.parametrize("n_heads,hd", [(5, 64), (4, 128), (30, 256), (8, 512)])
def test_rmsnorm_per_head_and_rope(ctx, eng, n_heads, hd):
    rng = np.random.default_rng(602 + hd)
    x = (rng.standard_normal(n_heads * hd) * 2).astype(np.float32)
    w = (1 + 0.2 * rng.standard_normal(hd)).astype(np.float32)
    tab = oracle.rope_table(9, hd, 10000.0, hd // 4)
    bx, bw, bt, y = ctx.buffer_f32(x), ctx.buffer_f32(w), ctx.buffer_f32(tab), ctx.buffer_empty_f32(n_heads * hd)
    eng.rmsnorm_per_head(ctx, n_heads, hd, 1e-6, bx, bw, y)
    assert_close(ctx.read_f32(y, n_heads * hd), oracle.rmsnorm_per_head(x, w, n_heads, hd, 1e-6), 1e-5, "norm")
    for pos in (0, 6):
        eng.rmsnorm_per_head_rope_off(ctx, n_heads, hd, 1e-6, bx, bw, bt, pos * hd, y)
        want = oracle.rmsnorm_per_head(x, w, n_heads, hd, 1e-6, tab[pos])
        assert_close(ctx.read_f32(y, n_heads * hd), want, 1e-5, f"rope row {pos}")
    # the position on the device, the whole table as input, in place
    meta = ctx.buffer_f32(np.array([7, 0, 0, 6], np.float32))
    k = eng._k(ctx, Kind.RMSNORM_PER_HEAD, (n_heads, hd, 2, 9), (), (1e-6,))
    ctx.encode_multi(k, [bx, bw, bt, meta], [bx])
    assert_close(ctx.read_f32(bx, n_heads * hd), want, 1e-5, "meta form, in place")
    with pytest.raises(hip.KshError, match="hd=96"):
        ctx.compile(hip.make_desc(Kind.RMSNORM_PER_HEAD, (2, 96, 0), (), (1e-6,)))


def test_add_scale_and_matvec_gelu_mul(ctx, eng):
    rng = np.random.default_rng(603)
    n = 7680
    a, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    ba, out = ctx.buffer_f32(a), ctx.buffer_empty_f32(n)
    eng.add_scale(ctx, n, 0.70710678, ba, ctx.buffer_f32(b), out)
    assert np.array_equal(ctx.read_f32(out, n), oracle.add_scale(a, b, 0.70710678))
    for rows, cols in ((256, 1536), (256, 2048), (10, 256), (64, 4608)):
        w = synth.q4k_blocks(rows * cols // 256, 604)
        x = rng.standard_normal(cols).astype(np.float32)
        cvec = rng.standard_normal(3 * rows).astype(np.float32)
        y = ctx.buffer_empty_f32(rows)
        eng.matvec_gelu_mul_at(ctx, rows, cols, DType.Q4K, ctx.buffer_bytes(w), ctx.buffer_f32(x), ctx.buffer_f32(cvec), 2 * rows, y)
        want = oracle.matvec_gelu_mul(oracle.Q4K, w, rows, cols, x, cvec[2 * rows:])
        assert_close(ctx.read_f32(y, rows), want, 1e-3, f"{rows}x{cols}")
    with pytest.raises(hip.KshError, match="Q4_K"):
        ctx.compile(hip.make_desc(Kind.MATVEC_GELU_MUL, (256, 2048), (DType.Q6K, DType.F32)))


def test_matvec_gelu_mul_closes_the_feed_forward_block(ctx, eng):
    """has_residual = 1: the gate GEMV computes x = res + rms(y)*w_post itself, multiplies against it and writes it."""
    rng = np.random.default_rng(605)
    for rows, cols in ((256, 1536), (256, 2048), (12, 512)):
        w = synth.q4k_blocks(rows * cols // 256, 606)
        y, res = (rng.standard_normal(cols) * 3).astype(np.float32), rng.standard_normal(cols).astype(np.float32)
        w_post = (1 + 0.2 * rng.standard_normal(cols)).astype(np.float32)
        cvec = rng.standard_normal(rows).astype(np.float32)
        u, x_new = ctx.buffer_empty_f32(rows), ctx.buffer_empty_f32(cols)
        k = eng._k(ctx, Kind.MATVEC_GELU_MUL, (rows, cols, 1), (DType.Q4K, DType.F32), (1e-6,))
        ctx.encode_multi(k, [ctx.buffer_bytes(w), ctx.buffer_f32(y), ctx.buffer_f32(cvec), ctx.buffer_f32(w_post), ctx.buffer_f32(res)], [u, x_new])
        want_x = oracle.rmsnorm(y, w_post, 1e-6, res=res)
        assert_close(ctx.read_f32(x_new, cols), want_x, 1e-5, "x_new")
        assert_close(ctx.read_f32(u, rows), oracle.matvec_gelu_mul(oracle.Q4K, w, rows, cols, want_x, cvec), 1e-3, f"{rows}x{cols}")


@pytest.mark.parametrize("wdt", [DType.Q4K, DType.Q6K])
def test_rmsnorm_matvec_stream_scale(ctx, eng, wdt):
    """params[1]: the folded-in add is RmsNormAddScale, x_new = scale * (res + rms(y)*w_post)."""
    rng = np.random.default_rng(607)
    rows, cols, scale = 512, 1536, 0.625
    w = (synth.q4k_blocks if wdt == DType.Q4K else synth.q6k_blocks)(rows * cols // 256, 608)
    y, res = (rng.standard_normal(cols) * 2).astype(np.float32), rng.standard_normal(cols).astype(np.float32)
    w_norm, w_post = ((1 + 0.2 * rng.standard_normal(cols)).astype(np.float32) for _ in range(2))
    out, x_new = ctx.buffer_empty_f32(rows), ctx.buffer_empty_f32(cols)
    k = eng._k(ctx, Kind.RMSNORM_MATVEC, (rows, cols, 1), (wdt, DType.F32), (1e-6, scale))
    ctx.encode_multi(k, [ctx.buffer_bytes(w), ctx.buffer_f32(y), ctx.buffer_f32(w_norm), ctx.buffer_f32(w_post), ctx.buffer_f32(res)], [out, x_new])
    want_x = oracle.rmsnorm(y, w_post, 1e-6, res=res, scale=scale)
    assert_close(ctx.read_f32(x_new, cols), want_x, 1e-5, "x_new")
    want = oracle.matvec(int(wdt), w, rows, cols, oracle.rmsnorm(want_x, w_norm, 1e-6))
    assert_close(ctx.read_f32(out, rows), want, 1e-3, "y")


PATTERN = [1, 1, 0, 1, 1, 1, 0, 1]
FFN = [1024, 1024, 2048, 1024, 1024, 1024, 2048, 1024]


@pytest.fixture(scope="module", params=["all_q4k", "mixed_q6k", "no_ple", "two_kv_heads", "wide_window"])
def tiny(ctx, request):
    cfg = dict(synth.GEMMA4_TINY)
    q6 = ()
    if request.param == "mixed_q6k":
        q6 = {(1, "wv"), (2, "wdown"), (3, "wq"), (4, "wgate"), (5, "wo"), (6, "wup"), (7, "proj")}
    if request.param == "no_ple":
        cfg["ple_dim"] = 0
    if request.param == "two_kv_heads":
        cfg["n_kv"] = 2                     # grouped-query attention: two q heads per kv head
    if request.param == "wide_window":
        cfg["sliding_window"] = 700         # longer than the short-context form takes: the merging attention on every layer
        cfg["max_seq"] = 800
    w = synth.gemma4_weights(cfg, 610, oracle.quantize_q4k, oracle.quantize_q6k, ffn=FFN, swa_pattern=PATTERN, q6k_tensors=q6, std=0.05)
    gpu, cpu = hip.Gemma4(ctx, cfg, w), oracle.Gemma4(cfg, w)
    yield gpu, cpu, cfg
    gpu.close()
    cpu.close()


def teacher_forced(gpu, cpu, cfg, pattern, toks, check=None, use_graph=False, tol=1e-3):
    """Feeds both models the same tokens with the oracle in lockstep: a K/V value on a Q4_0 rounding boundary may
    take the neighbouring code on two correct f32 implementations, so the oracle packs its own row in every
    cache-owning layer, checks that the device's row is within one code step of it and continues with the device's
    row (`adopt_rows`).  Both sides attend over identical caches in every layer, so every step is compared.
    Returns (steps compared, steps whose greedy token was checked and agreed)."""
    ctx = gpu.ctx
    n = cfg["n_layers"]
    owners = [l for l in range(n) if gpu.kv_source(l) == l]
    hd = {l: cfg["hd_swa"] if pattern[l] else cfg["hd_full"] for l in owners}
    bufs = {l: [hip.Buffer(ctx, hip.lib().ksh_gemma4_kv(gpu.h, l, w), owned=False) for w in (0, 1)] for l in owners}
    stride = max(cfg["n_kv"] * h // 32 * 18 for h in hd.values())
    agree = compared = flipped = 0
    for i, t in enumerate(toks):
        compare = check is None or i in check
        g_next = gpu.forward_token(int(t), want_logits=compare, use_graph=use_graph)
        rows = np.zeros((n, 2, stride), np.uint8)
        for l in owners:
            row = cfg["n_kv"] * hd[l] // 32 * 18
            for w in (0, 1):
                rows[l, w, :row] = ctx.read_bytes(bufs[l][w], row, i * row)
        c_next, c_logits = cpu.forward(int(t), want_logits=compare, return_logits=True, adopt_rows=rows)
        assert cpu.row_max_step.max() <= 1.0 + 1e-3, (i, cpu.row_max_step.max(1))      # a flip is one code step, never more
        flipped += int(cpu.row_diff_bytes.sum())
        if not compare:
            continue
        g_logits = gpu.logits()
        assert g_next == oracle.softcap_argmax(g_logits, cfg["softcap"])       # the device argmax follows the oracle's rule
        compared += 1
        assert_close(g_logits, c_logits, tol, f"logits at step {i}")
        assert_close(gpu.hidden(), cpu.hidden(), tol, f"hidden at step {i}")
        top2 = np.sort(c_logits)[-2:]
        if top2[1] - top2[0] > 2 * tol * max(abs(top2[1]), float(np.sqrt(np.mean(c_logits ** 2)))):
            assert g_next == c_next, f"step {i}: margin {top2[1] - top2[0]}"
            agree += 1
    assert flipped <= 0.02 * len(toks) * len(owners) * 2 * stride, flipped
    return compared, agree


def test_gemma4_forward_token_matches_oracle_teacher_forced(tiny):
    """24 positions: three times the sliding window."""
    gpu, cpu, cfg = tiny
    gpu.reset()
    cpu.reset()
    n_layers = cfg["n_layers"]
    assert [gpu.kv_source(l) for l in range(n_layers)] == [cpu.kv_source(l) for l in range(n_layers)] == [0, 1, 2, 3, 4, 4, 2, 4]
    toks = np.random.default_rng(611).integers(0, cfg["vocab"], 24)
    clean, agree = teacher_forced(gpu, cpu, cfg, PATTERN, toks)
    assert clean == len(toks) and agree >= 16 and gpu.pos == cpu.pos == len(toks), (clean, agree)
    with pytest.raises(hip.KshError, match="outside the vocabulary"):
        gpu.forward_token(cfg["vocab"])


def prefilled_in_lockstep(gpu, cpu, cfg, pattern, toks, then=4, tol=1e-3):
    """prefill_chunk(toks) as batched chunks, then the oracle walks the same positions adopting the rows the chunk
    left (one code step at most from its own), then `then` decode steps with logits compared."""
    ctx, n = gpu.ctx, cfg["n_layers"]
    owners = [l for l in range(n) if gpu.kv_source(l) == l]
    hd = {l: cfg["hd_swa"] if pattern[l] else cfg["hd_full"] for l in owners}
    stride = max(cfg["n_kv"] * h // 32 * 18 for h in hd.values())
    n_pre = len(toks) - then
    gpu.reset()
    cpu.reset()
    gpu.prefill_chunk(toks[:n_pre])
    assert gpu.pos == n_pre
    cache = {l: [gpu.kv(l, w, n_pre * (cfg["n_kv"] * hd[l] // 32 * 18)) for w in (0, 1)] for l in owners}
    flipped = 0
    for i in range(n_pre):
        rows = np.zeros((n, 2, stride), np.uint8)
        for l in owners:
            row = cfg["n_kv"] * hd[l] // 32 * 18
            for w in (0, 1):
                rows[l, w, :row] = cache[l][w][i * row:(i + 1) * row]
        cpu.forward(int(toks[i]), want_logits=False, adopt_rows=rows)
        assert cpu.row_max_step.max() <= 1.0 + 1e-3, (i, cpu.row_max_step.max(1))
        flipped += int(cpu.row_diff_bytes.sum())
    assert flipped <= 0.02 * n_pre * len(owners) * 2 * stride, flipped
    bufs = {l: [hip.Buffer(ctx, hip.lib().ksh_gemma4_kv(gpu.h, l, w), owned=False) for w in (0, 1)] for l in owners}
    for i in range(n_pre, len(toks)):
        g_next = gpu.forward_token(int(toks[i]), use_graph=bool(i & 1))
        rows = np.zeros((n, 2, stride), np.uint8)
        for l in owners:
            row = cfg["n_kv"] * hd[l] // 32 * 18
            for w in (0, 1):
                rows[l, w, :row] = ctx.read_bytes(bufs[l][w], row, i * row)
        c_next, c_logits = cpu.forward(int(toks[i]), return_logits=True, adopt_rows=rows)
        assert cpu.row_max_step.max() <= 1.0 + 1e-3
        assert_close(gpu.logits(), c_logits, tol, f"logits at position {i}")
        top2 = np.sort(c_logits)[-2:]
        if top2[1] - top2[0] > 2 * tol * max(abs(top2[1]), float(np.sqrt(np.mean(c_logits ** 2)))):
            assert g_next == c_next


@pytest.mark.parametrize("n_pre", [2, 7, 20, 37])
def test_gemma4_prefill_chunk_batched(tiny, n_pre):
    """The batched layer pass over a prompt chunk (both layer kinds, a window of 8 that the chunk outgrows, layers
    reading earlier caches, per-layer embeddings, Q4_K and Q6_K tensors): the KV rows of the serial run up to
    one-code flips, and the oracle's logits on the decode steps behind it."""
    gpu, cpu, cfg = tiny
    toks = np.random.default_rng(640 + n_pre).integers(0, cfg["vocab"], n_pre + 4)
    prefilled_in_lockstep(gpu, cpu, cfg, PATTERN, toks)
    # the same prompt through the decode step leaves the same position and (up to flips) the same cache
    batched = {l: gpu.kv(l, 0, 64) for l in range(cfg["n_layers"]) if gpu.kv_source(l) == l}
    gpu.reset()
    gpu.prefill_chunk(toks[:n_pre], serial=True)
    assert gpu.pos == n_pre
    for l, b in batched.items():
        assert (gpu.kv(l, 0, 64) != b).mean() <= 0.1


def test_gemma4_generate_graph_equals_eager_and_oracle(tiny):
    gpu, cpu, cfg = tiny
    prompt = [int(t) for t in np.random.default_rng(612).integers(0, cfg["vocab"], 6)]
    n_new = 30
    gpu.reset()
    eager, _, _ = gpu.generate(prompt, n_new, use_graph=False)
    gpu.reset()
    graph, _, _ = gpu.generate(prompt, n_new, use_graph=True)
    assert graph == eager
    gpu.reset()
    assert gpu.generate(prompt, n_new, use_graph=True)[0] == graph      # replay after reset
    assert gpu.launches_per_token > 0
    cpu.reset()
    for t in prompt[:-1]:
        cpu.forward(t, want_logits=False)
    want, tok = [], prompt[-1]
    margins = []
    for _ in range(n_new):
        tok, logits = cpu.forward(tok, return_logits=True)
        want.append(tok)
        top2 = np.sort(logits)[-2:]
        margins.append((top2[1] - top2[0]) / max(abs(top2[1]), 1e-6))
    # identical up to the first step whose top-2 margin is inside f32 reassociation noise
    first_close = next((i for i, mg in enumerate(margins) if mg < 1e-3), n_new)
    assert graph[:first_close] == want[:first_close]
    assert first_close >= 8
    with pytest.raises(hip.KshError, match="max_seq"):
        gpu.generate(prompt, cfg["max_seq"], use_graph=True)
    # the stop rule: the run ends with the first id from the list, which is the last id returned
    for stop_at in (0, 3, n_new - 1):
        eos = [graph[stop_at], cfg["vocab"] - 1]
        first = next(i for i, t in enumerate(graph) if t in eos)
        gpu.reset()
        got, _, _ = gpu.generate_until(prompt, n_new, eos=eos, use_graph=True)
        assert got == graph[:first + 1], stop_at
    gpu.reset()
    assert gpu.generate_until(prompt, n_new, eos=(), use_graph=False)[0] == graph     # nothing to stop at: the whole run


def test_gemma4_plans_are_warmed_at_load(ctx, tmp_path, monkeypatch):
    """The load warms one schedule search per distinct GEMV shape of the layers (gemma_prim.rs:254-290) unless
    KSEARCH_SKIP_BEAM is set: two feed-forward widths leave two plans each for the gate/up and the down kinds, a
    second load is served from the files, and the decode step under the planned schedules matches the oracle."""
    monkeypatch.setenv("KSEARCH_BEAM_CACHE", str(tmp_path / "beam"))
    monkeypatch.delenv("KSEARCH_SKIP_BEAM", raising=False)
    cfg = dict(synth.GEMMA4_TINY)
    w = synth.gemma4_weights(cfg, 612, oracle.quantize_q4k, oracle.quantize_q6k, ffn=FFN, swa_pattern=PATTERN, std=0.05)
    gpu, cpu = hip.Gemma4(ctx, cfg, w), oracle.Gemma4(cfg, w)
    names = sorted(f.name for f in (tmp_path / "beam").glob("*.txt"))
    assert sum(n.startswith("rms_matvec_gate_up_q4k") for n in names) == 2, names
    assert sum(n.startswith("rms_matvec_qkv_q4k") for n in names) >= 1 and sum(n.startswith("matvec_q4k") for n in names) >= 3, names
    stamp = {f.name: f.stat().st_mtime_ns for f in (tmp_path / "beam").glob("*.txt")}
    toks = np.random.default_rng(613).integers(0, cfg["vocab"], 6)
    compared, _ = teacher_forced(gpu, cpu, cfg, PATTERN, toks, use_graph=True)
    assert compared == 6
    gpu.close()
    again = hip.Gemma4(ctx, cfg, w)
    assert {f.name: f.stat().st_mtime_ns for f in (tmp_path / "beam").glob("*.txt")} == stamp
    again.close()
    cpu.close()


def test_gemma4_create_errors(ctx):
    cfg = dict(synth.GEMMA4_TINY, vocab=256)
    w = synth.gemma4_weights(cfg, 613, oracle.quantize_q4k, oracle.quantize_q6k, ffn=512, swa_pattern=PATTERN)
    with pytest.raises(hip.KshError, match="invalid configuration"):
        hip.Gemma4(ctx, dict(cfg, shared_kv_layers=8), w)
    # the reference's default pattern has no owning full-attention layer among the first five: the sixth layer
    # would read a cache of another head dim
    w_bad = synth.gemma4_weights(cfg, 613, oracle.quantize_q4k, oracle.quantize_q6k, ffn=512)
    with pytest.raises(hip.KshError, match="another head dim"):
        hip.Gemma4(ctx, cfg, w_bad)
    gone = dict(w, layers=[{k: v for k, v in w["layers"][0].items() if k != "post_norm"}] + w["layers"][1:])
    with pytest.raises(hip.KshError, match="per-layer-embedding weights are missing"):
        hip.Gemma4(ctx, cfg, gone)
    bad = dict(w, layers=[dict(w["layers"][0], dt_q=int(DType.Q5K))] + w["layers"][1:])
    with pytest.raises(hip.KshError, match="weight dtype"):
        hip.Gemma4(ctx, cfg, bad)


def test_gemma4_from_gguf_matches_oracle(ctx, tmp_path):
    """A GGUF file with the tensor names, types and metadata keys of the real checkpoints: Q4_K and Q6_K
    matrices, f32 norms, an f32 per-layer model projection (scaled by 1/sqrt(hidden) and packed at load), an f16
    per-layer gate and a bf16 projection (packed at load), a Q5_K per-layer table, a Q6_K ffn_down (requantized
    to Q4_K like the reference does) beside a Q6_K attn_q (kept).  The oracle gets the same tensors converted by
    the host routines."""
    from tests import gguf_writer as gw
    from ksearch_amd.hip import GgmlType
    cfg = dict(synth.GEMMA4_TINY)
    n, h, pd = cfg["n_layers"], cfg["hidden"], cfg["ple_dim"]
    w = synth.gemma4_weights(cfg, 620, oracle.quantize_q4k, oracle.quantize_q6k, ffn=FFN, swa_pattern=PATTERN,
                             q6k_tensors={(2, "wdown"), (3, "wq")}, std=0.05)
    rng = np.random.default_rng(621)
    names = dict(wq="attn_q", wk="attn_k", wv="attn_v", wo="attn_output", wgate="ffn_gate", wup="ffn_up", wdown="ffn_down",
                 attn_norm="attn_norm", q_norm="attn_q_norm", k_norm="attn_k_norm", post_attn_norm="post_attention_norm", ffn_norm="ffn_norm",
                 post_ffw_norm="post_ffw_norm", post_norm="post_norm")
    dt2ggml = {oracle.Q4K: GgmlType.Q4_K, oracle.Q6K: GgmlType.Q6_K}
    tensors = []
    for i, lw in enumerate(w["layers"]):
        hd = cfg["hd_swa"] if lw["is_swa"] else cfg["hd_full"]
        cols = dict(wq=h, wk=h, wv=h, wo=cfg["n_q"] * hd, wgate=h, wup=h, wdown=lw["ffn"])
        for key, dtk in (("wq", "dt_q"), ("wk", "dt_k"), ("wv", "dt_v"), ("wo", "dt_o"), ("wgate", "dt_gate"), ("wup", "dt_up"), ("wdown", "dt_down")):
            if key not in lw:
                continue
            blk = 144 if lw[dtk] == oracle.Q4K else 210
            rows = lw[key].size // blk * 256 // cols[key]
            tensors.append((f"blk.{i}.{names[key]}.weight", dt2ggml[lw[dtk]], (cols[key], rows), lw[key]))
        for key in ("attn_norm", "q_norm", "k_norm", "post_attn_norm", "ffn_norm", "post_ffw_norm", "post_norm"):
            tensors.append((f"blk.{i}.{names[key]}.weight", GgmlType.F32, (lw[key].size,), lw[key]))
        tensors.append((f"blk.{i}.layer_output_scale.weight", GgmlType.F32, (1,), np.array([lw["layer_scale"]], np.float32)))
        # per-layer gate in f16, projection in bf16: both are packed to Q4_K by the loader
        gate = (rng.standard_normal(pd * h) * 0.05).astype(np.float16)
        proj32 = (rng.standard_normal(h * pd) * 0.05).astype(np.float32)
        proj = (proj32.view(np.uint32) >> 16).astype(np.uint16)
        tensors.append((f"blk.{i}.inp_gate.weight", GgmlType.F16, (h, pd), gate))
        tensors.append((f"blk.{i}.proj.weight", GgmlType.BF16, (pd, h), proj))
        lw["inp_gate"], lw["dt_inp_gate"] = oracle.quantize_q4k(gate.astype(np.float32)), oracle.Q4K
        lw["proj"], lw["dt_proj"] = oracle.quantize_q4k((proj.astype(np.uint32) << 16).view(np.float32)), oracle.Q4K
        if lw["dt_down"] == oracle.Q6K:      # gemma_prim.rs:418-433
            lw["wdown"], lw["dt_down"] = oracle.quantize_q4k(oracle.dequant(oracle.Q6K, lw["wdown"], h * lw["ffn"])), oracle.Q4K
    g = w["globals"]
    pt = n * pd
    model_proj = (rng.standard_normal(pt * h) * 0.05).astype(np.float32)
    tensors += [("token_embd.weight", GgmlType.Q6_K, (h, cfg["vocab"]), g["token_embd"]), ("output_norm.weight", GgmlType.F32, (h,), g["output_norm"]),
                ("per_layer_token_embd.weight", GgmlType.Q5_K, (pt, cfg["vocab"]), g["ple_embd"]),
                ("per_layer_model_proj.weight", GgmlType.F32, (h, pt), model_proj),
                ("per_layer_proj_norm.weight", GgmlType.F32, (pd,), g["ple_proj_norm"])]
    g["ple_model_proj"] = oracle.quantize_q4k(model_proj * np.float32(1.0 / np.sqrt(np.float32(h))))      # :341-352
    meta = [("general.architecture", gw.STR, "gemma4"), ("gemma4.block_count", gw.U32, n), ("gemma4.embedding_length", gw.U32, h),
            ("gemma4.attention.head_count", gw.U32, cfg["n_q"]), ("gemma4.attention.head_count_kv", gw.U32, cfg["n_kv"]),
            ("gemma4.attention.key_length", gw.U32, cfg["hd_full"]), ("gemma4.attention.key_length_swa", gw.U32, cfg["hd_swa"]),
            ("gemma4.attention.sliding_window", gw.U32, cfg["sliding_window"]), ("gemma4.attention.shared_kv_layers", gw.U32, cfg["shared_kv_layers"]),
            ("gemma4.embedding_length_per_layer_input", gw.U32, pd), ("gemma4.feed_forward_length", gw.ARR, (gw.U32, FFN)),
            ("gemma4.attention.sliding_window_pattern", gw.ARR, (gw.BOOL, PATTERN))]
    path = str(tmp_path / "tiny.gguf")
    gw.write(path, meta, tensors)
    with hip.Gguf(path) as f:
        gpu = hip.Gemma4.from_gguf(ctx, f, cfg["max_seq"])
    for k in ("n_layers", "hidden", "vocab", "hd_swa", "hd_full", "sliding_window", "shared_kv_layers", "ple_dim", "attn_scale"):
        assert gpu.cfg[k] == cfg[k], k
    cpu = oracle.Gemma4(cfg, w)
    prompt = [int(t) for t in np.random.default_rng(622).integers(0, cfg["vocab"], 5)]
    got, _, _ = gpu.generate(prompt, 24, use_graph=True)
    for t in prompt[:-1]:
        cpu.forward(t, want_logits=False)
    want, tok, margins = [], prompt[-1], []
    for _ in range(24):
        tok, logits = cpu.forward(tok, return_logits=True)
        want.append(tok)
        top2 = np.sort(logits)[-2:]
        margins.append((top2[1] - top2[0]) / max(abs(top2[1]), 1e-6))
    first_close = next((i for i, mg in enumerate(margins) if mg < 1e-3), 24)
    assert got[:first_close] == want[:first_close] and first_close >= 8
    gpu.close()
    cpu.close()
    # the same file with the Q6_K ffn_down kept: a different (closer) model, so not the reference's tokens in general,
    # but the loader must take it
    with hip.Gguf(path) as f:
        kept = hip.Gemma4.from_gguf(ctx, f, cfg["max_seq"], keep_q6k=True)
    assert len(kept.generate(prompt, 4, use_graph=False)[0]) == 4
    kept.close()
    # a tensor whose shape contradicts the metadata
    bad = [(nm, ty, ((dims[0], dims[1] - 1) if nm == "blk.0.attn_q.weight" else dims), (raw[:-(h // 256 * 144)] if nm == "blk.0.attn_q.weight" else raw))
           for nm, ty, dims, raw in tensors]
    gw.write(path, meta, bad)
    with hip.Gguf(path) as f, pytest.raises(hip.KshError, match="blk.0.attn_q.weight is"):
        hip.Gemma4.from_gguf(ctx, f, cfg["max_seq"])


def real_widths_models(ctx, eng):
    """The real checkpoints' widths (hidden 1536, head dims 256 / 512, window 512, double-wide feed-forward on the
    layers that reuse a cache, unscaled attention) on a shortened stack; the oracle on the very same packed bytes
    (quantized on the device, read back for the CPU)."""
    n, shared = 9, 4
    cfg = dict(n_layers=n, hidden=1536, n_q=8, n_kv=1, vocab=8192, max_seq=576, hd_swa=256, hd_full=512, sliding_window=512,
               shared_kv_layers=shared, ple_dim=256, eps=1e-6, softcap=30.0, rope_theta_swa=1e4, rope_theta_full=1e6,
               partial_rotary=0.25, attn_scale=1.0)
    pattern = [1, 1, 0, 1, 1, 1, 1, 0, 1]          # owners 0..4 (full: 2); 5, 6, 8 read layer 4's cache, 7 reads layer 2's
    ffn = [6144 if i < n - shared else 12288 for i in range(n)]
    dq4, dq6 = hip.device_quantizers(ctx, eng)
    dev = synth.gemma4_weights(cfg, 630, dq4, lambda x: dq6([x]), ffn=ffn, swa_pattern=pattern, std=0.05)

    def host(v):
        return ctx.read_bytes(v, v.nbytes) if isinstance(v, hip.Buffer) else v

    w = dict(layers=[{k: host(v) for k, v in lw.items()} for lw in dev["layers"]], globals={k: host(v) for k, v in dev["globals"].items()})
    gpu, cpu = hip.Gemma4(ctx, cfg, dev), oracle.Gemma4(cfg, w)
    cpu.host_weights = w                # (for a second oracle over the same bytes)
    assert [gpu.kv_source(l) for l in range(n)] == [0, 1, 2, 3, 4, 4, 4, 2, 4]
    return gpu, cpu, cfg, pattern


def test_gemma4_real_widths_batched_prefill(ctx, eng):
    """300 prompt tokens at the real widths as one chunk (512-wide heads, 12288-wide feed-forward, 1536-column GEMMs,
    the per-layer table; the 256-wide heads' attention on the matrix cores), then decode steps against the oracle.
    The chunk itself is held to "every K / V row within one code step of the oracle's" inside the helper.  The bar
    on the decode steps' logits is 1e-2: with unscaled scores over 300 rows the softmax is close to one-hot, and
    which position shows the largest difference depends on the rows the chunk left -- over three seeds and both
    forms of the chunk's attention the per-position maximum ran from 1e-4 to 6e-3, with one position per seed
    above 2e-3."""
    gpu, cpu, cfg, pattern = real_widths_models(ctx, eng)
    toks = np.random.default_rng(632).integers(0, cfg["vocab"], 304)
    prefilled_in_lockstep(gpu, cpu, cfg, pattern, toks, then=4, tol=1e-2)
    gpu.close()
    cpu.close()


def test_gemma4_real_widths_long_run_matches_oracle(ctx, eng):
    """The real checkpoints' widths (hidden 1536, head dims 256 / 512, window 512, double-wide feed-forward on the
    layers that reuse a cache, unscaled attention) on a shortened stack, teacher-forced past the window through
    the captured graph, against the oracle on the very same packed bytes (quantized on the device, read back for
    the CPU).  Logits are compared where the run changes regime: the first positions, the oracle's switch to
    split-KV attention at 128 rows, the window's edge at 512.  The bar is 1e-2 on whole-model logits here, as in the
    batched-prefill test above: with unscaled scores over hundreds of rows of random weights the softmax is close to
    one-hot, and an f32 difference in the last bit of a score (a different association, a product contracted into an
    fma or not) moves the output by more than it does at the tiny model's 24 rows (1e-3 there; the single ops stay at
    1e-3 in their own tests).  Measured, per-position maximum over 63 positions, for two instances of the attention
    step that differ in nothing but such last bits (their partitions agree to 7e-6) and two token seeds: 3.5e-3 and
    8.8e-3 (seed 631), 5.4e-3 and 4.1e-3 (seed 632), each at a different position; the median position is at 6e-4."""
    gpu, cpu, cfg, pattern = real_widths_models(ctx, eng)
    toks = np.random.default_rng(631).integers(0, cfg["vocab"], 540)
    check = set(range(12)) | set(range(124, 134)) | set(range(506, 520)) | {300, 539}
    clean, agree = teacher_forced(gpu, cpu, cfg, pattern, toks, check=check, use_graph=True, tol=1e-2)
    assert clean == len(check) and agree >= 0.5 * len(check), (clean, agree)
    gpu.close()
    cpu.close()


def test_kvpool_slot_rules(ctx):
    """kv_pool.rs:232-248 restated (first free slot, a freed slot is reused), the bump and bounds rules, clear_slot."""
    pool = hip.KvPool(ctx, 4, 64, 2, 256, 1)
    a, b = pool.alloc(), pool.alloc()
    assert a != b and len(pool.active_batch()) == 2
    pool.free(a)
    assert pool.active_batch() == [b]
    assert pool.alloc() == a
    assert pool.bump_len(a, 5) == 5 and pool.bump_len(a) == 6 and pool.seq_len(a) == 6 and pool.seq_len(b) == 0
    with pytest.raises(hip.KshError, match="slot seq full"):
        pool.bump_len(a, 59)
    pool.alloc(), pool.alloc()
    with pytest.raises(hip.KshError, match=r"KvPool full \(max_batch=4\)"):
        pool.alloc()
    pool.free(b)
    with pytest.raises(hip.KshError, match="slot not occupied"):
        pool.bump_len(b)
    with pytest.raises(hip.KshError, match="bad SlotId"):
        pool.free(9)
    assert pool.seq_len(9) == -1
    nbytes = 64 * 1 * 8 * 18
    ctx.write_bytes(pool.k_buf(a, 1), np.full(nbytes, 0xAB, np.uint8))
    pool.clear_slot(a)
    assert not ctx.read_bytes(pool.k_buf(a, 1), nbytes).any() and pool.k_buf(a, 1).nbytes == nbytes
    pool.close()
    with pytest.raises(hip.KshError, match="non-zero"):
        hip.KvPool(ctx, 0, 64, 2, 256, 1)


def test_gemma4_two_sequences_interleaved_through_pool_slots(tiny):
    """One model, two sequences in two pool slots, advanced in turn (bind_slot, one token, bump): each produces the
    tokens it produces alone, through the captured per-slot graphs and eagerly; then the model goes back to its own
    caches."""
    gpu, _, cfg = tiny
    ctx = gpu.ctx
    rng = np.random.default_rng(640)
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab"], n)] for n in (5, 9)]
    n_new = 14
    alone = []
    for p in prompts:
        gpu.bind_slot(None, 0)
        gpu.reset()
        alone.append(gpu.generate(p, n_new, use_graph=True)[0])
    owners = cfg["n_layers"] - cfg["shared_kv_layers"]
    pool = hip.KvPool(ctx, 3, cfg["max_seq"], owners, max(cfg["hd_swa"], cfg["hd_full"]), cfg["n_kv"])
    for use_graph in (True, False):
        slots = [pool.alloc(), pool.alloc()]
        for s_ in slots:
            pool.clear_slot(s_)
        feed = [list(p) for p in prompts]           # tokens still to be fed; the last fed token's successor is appended
        outs = [[], []]
        while any(len(o) < n_new for o in outs):
            for i, s_ in enumerate(slots):
                if len(outs[i]) >= n_new:
                    continue
                gpu.bind_slot(pool, s_)
                assert gpu.pos == pool.seq_len(s_)
                tok = feed[i].pop(0)
                last_of_prompt = not feed[i]
                nxt = gpu.forward_token(tok, want_logits=last_of_prompt, use_graph=use_graph)
                pool.bump_len(s_)
                if last_of_prompt:
                    outs[i].append(nxt)
                    feed[i].append(nxt)
        assert outs == alone, use_graph
        for s_ in slots:
            pool.free(s_)
    with pytest.raises(hip.KshError, match="kv layer mismatch"):
        gpu.bind_slot(hip.KvPool(ctx, 1, cfg["max_seq"], owners + 1, 256, cfg["n_kv"]), 0)
    with pytest.raises(hip.KshError, match="bad SlotId"):
        gpu.bind_slot(pool, 7)
    gpu.bind_slot(None, 0)
    gpu.reset()
    assert gpu.generate(prompts[0], n_new, use_graph=True)[0] == alone[0]
    pool.close()


def slot_rows(ctx, pool, slot, pos, cfg, pattern, owners):
    """The K / V rows position `pos` left in a pool slot, one per cache-owning layer, padded to the widest."""
    n = cfg["n_layers"]
    hd = {l: cfg["hd_swa"] if pattern[l] else cfg["hd_full"] for l in owners}
    stride = max(cfg["n_kv"] * h // 32 * 18 for h in hd.values())
    rows = np.zeros((n, 2, stride), np.uint8)
    for l in owners:
        row = cfg["n_kv"] * hd[l] // 32 * 18
        rows[l, 0, :row] = ctx.read_bytes(pool.k_buf(slot, l), row, pos * row)
        rows[l, 1, :row] = ctx.read_bytes(pool.v_buf(slot, l), row, pos * row)
    return rows


@pytest.mark.parametrize("variant", ["all_q4k", "mixed_q6k_two_kv_heads"])
def test_gemma4_decode_round_over_pool_slots(ctx, variant):
    """One decode step for several sequences as one pass over the weights (the scheduler's decode round,
    crates/ksearch_cli/src/scheduler.rs:163-231, there one step per request).  Three sequences of different lengths in
    slots 2, 0 and 3 of a four-slot pool (prompts fed through bind_slot + prefill_chunk), then 12 rounds of all three
    (across the sliding window's edge), one of two of them, and serial steps in between; each sequence has its own
    oracle, walking the same tokens in lockstep with the rows its slot received: every row's logits within 1e-3, the
    greedy id the oracle's where its margin allows, appended K / V rows within one code of the oracle's."""
    cfg = dict(synth.GEMMA4_TINY)
    q6 = ()
    if variant != "all_q4k":
        cfg["n_kv"] = 2
        q6 = {(1, "wv"), (2, "wdown"), (3, "wq"), (4, "wgate"), (5, "wo"), (6, "wup"), (7, "proj")}
    w = synth.gemma4_weights(cfg, 651, oracle.quantize_q4k, oracle.quantize_q6k, ffn=FFN, swa_pattern=PATTERN, q6k_tensors=q6, std=0.05)
    gpu = hip.Gemma4(ctx, cfg, w)
    n, tol = cfg["n_layers"], 1e-3
    owners = [l for l in range(n) if gpu.kv_source(l) == l]
    pool = hip.KvPool(ctx, 4, cfg["max_seq"], len(owners), max(cfg["hd_swa"], cfg["hd_full"]), cfg["n_kv"])
    for _ in range(4):
        pool.clear_slot(pool.alloc())
    pool.free(1)
    rng = np.random.default_rng(650)
    slots, pre = [2, 0, 3], [5, 1, 11]
    cpus = [oracle.Gemma4(cfg, w) for _ in slots]           # one oracle per sequence
    try:
        for cpu in cpus:
            cpu.reset()
        for s_, n_pre, cpu in zip(slots, pre, cpus):
            toks = [int(t) for t in rng.integers(0, cfg["vocab"], n_pre)]
            gpu.bind_slot(pool, s_)
            gpu.prefill_chunk(toks)
            pool.bump_len(s_, n_pre)
            for i, t in enumerate(toks):
                cpu.forward(t, want_logits=False, adopt_rows=slot_rows(ctx, pool, s_, i, cfg, PATTERN, owners))
                assert cpu.row_max_step.max() <= 1.0 + 1e-3
        checked = 0

        def check_rows(active, toks, nxt, logits):
            nonlocal checked
            for j, i in enumerate(active):
                pos = pool.seq_len(slots[i])
                c_next, c_logits = cpus[i].forward(int(toks[j]), return_logits=True, adopt_rows=slot_rows(ctx, pool, slots[i], pos, cfg, PATTERN, owners))
                assert cpus[i].row_max_step.max() <= 1.0 + 1e-3, (i, pos)
                assert_close(logits[j], c_logits, tol, f"sequence {i} at position {pos}")
                assert nxt[j] == oracle.softcap_argmax(logits[j], cfg["softcap"])
                top2 = np.sort(c_logits)[-2:]
                if top2[1] - top2[0] > 2 * tol * max(abs(top2[1]), float(np.sqrt(np.mean(c_logits ** 2)))):
                    assert nxt[j] == c_next
                    checked += 1
                pool.bump_len(slots[i])

        for r in range(12):
            toks = rng.integers(0, cfg["vocab"], 3)
            nxt = gpu.decode_round(pool, slots, toks)
            check_rows([0, 1, 2], toks, nxt, gpu.round_logits(3))
            if r == 5:
                # a serial step on one of the slots in between: bind_slot finds the slot's length moved and re-seeks
                gpu.bind_slot(pool, slots[1])
                assert gpu.pos == pool.seq_len(slots[1])
                t = int(rng.integers(0, cfg["vocab"]))
                g_next = gpu.forward_token(t, want_logits=True, use_graph=True)
                check_rows([1], [t], [g_next], gpu.logits()[None, :])
        toks = rng.integers(0, cfg["vocab"], 2)
        nxt = gpu.decode_round(pool, [slots[2], slots[0]], toks)          # a subset, in another order
        check_rows([2, 0], toks, nxt, gpu.round_logits(2))
        nxt = gpu.decode_round(pool, [slots[1]], [7])                      # a round of one
        check_rows([1], [7], nxt, gpu.round_logits(1))
        assert checked >= 20
        # sampled rows: the host sampler's draw on that row's logits
        toks = rng.integers(0, cfg["vocab"], 3)
        nxt = gpu.decode_round(pool, slots, toks, temperature=[0.0, 0.8, 1.3], min_p=[0.0, 0.05, 0.0], seeds=[1, 77, 991])
        lg = gpu.round_logits(3)
        assert nxt[0] == oracle.softcap_argmax(lg[0], cfg["softcap"])
        assert nxt[1] == hip.sample_softcap_min_p(lg[1], cfg["softcap"], 0.8, 0.05, 77)
        assert nxt[2] == hip.sample_softcap_min_p(lg[2], cfg["softcap"], 1.3, 0.0, 991)
        # errors
        with pytest.raises(hip.KshError, match="named twice"):
            gpu.decode_round(pool, [0, 0], [1, 2])
        with pytest.raises(hip.KshError, match="slot not occupied"):
            gpu.decode_round(pool, [1, 0], [1, 2])
        with pytest.raises(hip.KshError, match="bad SlotId"):
            gpu.decode_round(pool, [9], [1])
        with pytest.raises(hip.KshError, match="outside the vocabulary"):
            gpu.decode_round(pool, [0], [cfg["vocab"]])
        with pytest.raises(hip.KshError, match="1 to 16"):
            gpu.decode_round(pool, list(range(17)), [1] * 17)
    finally:
        for cpu in cpus:
            cpu.close()
        gpu.close()
        pool.close()


def test_gemma4_decode_round_after_the_pool_is_replaced(ctx):
    """The per-width round graphs hold the pool's device addresses.  A pool that is destroyed and replaced (the host
    object of the new one may well come up at the old one's address, its layers elsewhere) must get graphs of its own:
    two rounds on the first pool (the second captures the width's graph), the pool closed, a larger one opened, then
    three rounds on it in lockstep with one oracle per sequence."""
    cfg = dict(synth.GEMMA4_TINY)
    w = synth.gemma4_weights(cfg, 652, oracle.quantize_q4k, oracle.quantize_q6k, ffn=FFN, swa_pattern=PATTERN, std=0.05)
    gpu = hip.Gemma4(ctx, cfg, w)
    n, tol = cfg["n_layers"], 1e-3
    owners = [l for l in range(n) if gpu.kv_source(l) == l]
    rng = np.random.default_rng(653)
    cpus = []
    pool = None
    try:
        for n_slots in (2, 5):
            pool = hip.KvPool(ctx, n_slots, cfg["max_seq"], len(owners), max(cfg["hd_swa"], cfg["hd_full"]), cfg["n_kv"])
            slots = [pool.alloc() for _ in range(n_slots)][-2:]
            for s_ in slots:
                pool.clear_slot(s_)
            cpus = [oracle.Gemma4(cfg, w) for _ in slots]
            for s_, n_pre, cpu in zip(slots, (3, 6), cpus):
                cpu.reset()
                toks = [int(t) for t in rng.integers(0, cfg["vocab"], n_pre)]
                gpu.bind_slot(pool, s_)
                gpu.prefill_chunk(toks)
                pool.bump_len(s_, n_pre)
                for i, t in enumerate(toks):
                    cpu.forward(t, want_logits=False, adopt_rows=slot_rows(ctx, pool, s_, i, cfg, PATTERN, owners))
            for r in range(3):
                toks = rng.integers(0, cfg["vocab"], 2)
                gpu.decode_round(pool, slots, toks)
                logits = gpu.round_logits(2)
                for j, s_ in enumerate(slots):
                    pos = pool.seq_len(s_)
                    _, c_logits = cpus[j].forward(int(toks[j]), return_logits=True, adopt_rows=slot_rows(ctx, pool, s_, pos, cfg, PATTERN, owners))
                    assert cpus[j].row_max_step.max() <= 1.0 + 1e-3, (n_slots, r, j)
                    assert_close(logits[j], c_logits, tol, f"pool of {n_slots}, round {r}, sequence {j}")
                    pool.bump_len(s_)
            for cpu in cpus:
                cpu.close()
            cpus = []
            gpu.bind_slot(None, 0)
            pool.close()
            pool = None
            junk = ctx.buffer_empty_f32(300_000)   # moves the next pool's layers off the old ones' addresses
    finally:
        for cpu in cpus:
            cpu.close()
        gpu.close()
        if pool is not None:
            pool.close()


def test_gemma4_real_widths_decode_round(ctx, eng):
    """Decode rounds at the real widths (hidden 1536, heads of 256 / 512, window 512, 12288-wide feed-forward): two
    sequences of 300 and 20 positions in slots 1 and 0 of a pool sized for the 512-wide heads (so the 256-wide layers'
    caches use half of each slot's stride), six rounds in lockstep with one oracle per sequence.  Bar: 5e-3 for the
    short sequence, as for the other runs at these widths; 2e-2 for the one that attends 300 rows, where the unscaled
    scores make the softmax nearly one-hot and a reordering of f32 sums moves single logits by several 1e-3 (the
    serial step on the same positions: up to 3.5e-3; the rounds: up to 9.6e-3)."""
    gpu, cpu_a, cfg, pattern = real_widths_models(ctx, eng)
    n = cfg["n_layers"]
    owners = [l for l in range(n) if gpu.kv_source(l) == l]
    pool = hip.KvPool(ctx, 3, cfg["max_seq"], len(owners), 512, cfg["n_kv"])
    slots, pre = [1, 0], [300, 20]
    for _ in range(2):
        pool.clear_slot(pool.alloc())
    rng = np.random.default_rng(660)
    # the second sequence's oracle: the same packed bytes, read back from the device like the first's
    cpu_b = oracle.Gemma4(cfg, cpu_a.host_weights)
    cpus = [cpu_a, cpu_b]
    try:
        for s_, n_pre, cpu in zip(slots, pre, cpus):
            cpu.reset()
            toks = [int(t) for t in rng.integers(0, cfg["vocab"], n_pre)]
            gpu.bind_slot(pool, s_)
            gpu.prefill_chunk(toks)
            pool.bump_len(s_, n_pre)
            for i, t in enumerate(toks):
                cpu.forward(t, want_logits=False, adopt_rows=slot_rows(ctx, pool, s_, i, cfg, pattern, owners))
                assert cpu.row_max_step.max() <= 1.0 + 1e-3, (s_, i)
        for r in range(6):
            toks = rng.integers(0, cfg["vocab"], 2)
            nxt = gpu.decode_round(pool, slots, toks)
            lg = gpu.round_logits(2)
            for j in range(2):
                pos = pool.seq_len(slots[j])
                _, c_logits = cpus[j].forward(int(toks[j]), return_logits=True, adopt_rows=slot_rows(ctx, pool, slots[j], pos, cfg, pattern, owners))
                assert cpus[j].row_max_step.max() <= 1.0 + 1e-3, (j, pos)
                assert_close(lg[j], c_logits, 2e-2 if pos >= 64 else 5e-3, f"sequence {j} at position {pos}")
                assert nxt[j] == oracle.softcap_argmax(lg[j], cfg["softcap"])
                pool.bump_len(slots[j])
    finally:
        cpu_b.close()
        cpu_a.close()
        gpu.close()
        pool.close()
