"""The decode chain (ksearch_amd/csrc/decode_chain.hip; KSEARCH_DECODE_CHAIN=1): a layer's o-projection, feed-forward
and the next layer's QKV as one launch whose phases hand their vectors to each other through memory.  Same
arithmetic as the four launches it replaces (gemma_prim.rs:1062-1197, :946-961), so it is held to the same parity:
the oracle in lockstep, and the launch-per-phase loop on the same weights."""
import numpy as np
import pytest

import oracle
from ksearch_amd import hip, synth
from tests.gpu_util import assert_close, rel_err

pytestmark = pytest.mark.gpu


def chain_cfg(n_layers):
    # the widths the chain is built for (the benchmark shape's), on a short stack and a small vocabulary
    return dict(n_layers=n_layers, hidden=2048, ffn=8192, n_q=8, n_kv=1, hd=256, vocab=4096, max_seq=1024,
                eps=1e-6, softcap=30.0, rope_theta=10000.0, attn_scale=1.0 / 16.0)


@pytest.fixture(scope="module")
def ctx():
    c = hip.Context()
    yield c
    c.close()


@pytest.mark.parametrize("n_layers", [4, 3])
def test_decode_chain_matches_the_oracle_and_the_separate_launches(ctx, monkeypatch, n_layers):
    """Both forms of the o-projection's input (the attention launch's unmerged partitions below the short-context
    limit, its merged output above), eager and replayed as a graph, an even and an odd number of layers (the two
    sets of hand-over vectors alternate per launch; an odd stack refills them between tokens)."""
    cfg = chain_cfg(n_layers)
    w = synth.gemma_weights(cfg, 900 + n_layers, oracle.quantize_q4k, synth.chunked(oracle.quantize_q6k), std=0.03)
    rng = np.random.default_rng(901)
    for lw in w["layers"]:
        for name in ("attn_norm", "q_norm", "k_norm", "post_attn_norm", "ffn_norm", "post_ffw_norm"):
            lw[name] = (1.0 + 0.2 * rng.standard_normal(lw[name].size)).astype(np.float32)
    monkeypatch.setenv("KSEARCH_SHORT_CONTEXT", "6")
    monkeypatch.setenv("KSEARCH_DECODE_CHAIN", "0")
    ref = hip.Gemma(ctx, cfg, w)
    monkeypatch.setenv("KSEARCH_DECODE_CHAIN", "1")
    gpu = hip.Gemma(ctx, cfg, w)
    cpu = oracle.Gemma(cfg, w)
    row = cfg["n_kv"] * cfg["hd"] // 32 * 18
    bufs = [[hip.Buffer(ctx, hip.lib().ksh_gemma_kv(gpu.h, l, x), owned=False) for x in (0, 1)] for l in range(n_layers)]
    try:
        toks = [int(t) for t in rng.integers(0, cfg["vocab"], 14)]
        for i, t in enumerate(toks):
            ref.forward_token(t, use_graph=False)
            g_next = gpu.forward_token(t, use_graph=bool(i & 1))
            g_logits = gpu.logits()
            rows = np.stack([np.stack([ctx.read_bytes(bufs[l][x], row, i * row) for x in (0, 1)]) for l in range(n_layers)])
            c_next, c_logits = cpu.forward(t, return_logits=True, adopt_rows=rows)
            assert cpu.row_max_step.max() <= 1.0 + 1e-3, i
            assert_close(g_logits, c_logits, 1e-3, f"step {i} against the oracle")
            if i == 0:
                # the same sums in another order (later positions attend caches that two runs fill independently,
                # where a value on a Q4_0 rounding boundary may take either code)
                assert float(rel_err(g_logits, ref.logits()).max()) <= 2e-4
            assert g_next == oracle.softcap_argmax(g_logits, cfg["softcap"])
            top2 = np.sort(c_logits)[-2:]
            if top2[1] - top2[0] > 2e-3 * max(abs(top2[1]), float(np.sqrt(np.mean(c_logits ** 2)))):
                assert g_next == c_next, i
        # one launch per layer instead of four: first QKV, (attention, chain) per layer, LM head, argmax + tail
        assert gpu.launches_per_token == 2 * n_layers + 4 + (n_layers & 1)
        # generate: prompt as a batched chunk (not the chain's business), then the chain token by token from a graph
        gpu.reset()
        a, _, _ = gpu.generate(toks[:9], 12, use_graph=True)
        gpu.reset()
        c, _, _ = gpu.generate(toks[:9], 12, use_graph=False)
        assert a == c and len(a) == 12
    finally:
        cpu.close()
        gpu.close()
        ref.close()


def test_decode_chain_wait_that_runs_out_is_an_error_not_a_hang(ctx, monkeypatch):
    """With a spin limit of zero every hand-over that is not there at the first look gives up: the launch still
    drains, the flag comes back as an error, and the model works again after a reset."""
    cfg = chain_cfg(2)
    w = synth.gemma_weights(cfg, 910, oracle.quantize_q4k, synth.chunked(oracle.quantize_q6k), std=0.03)
    monkeypatch.setenv("KSEARCH_DECODE_CHAIN", "1")
    monkeypatch.setenv("KSEARCH_CHAIN_SPIN_LIMIT", "0")
    bad = hip.Gemma(ctx, cfg, w)
    with pytest.raises(hip.KshError, match="hand-over wait ran out"):
        for t in range(4):
            bad.forward_token(5 + t, use_graph=False)
    bad.close()
    monkeypatch.delenv("KSEARCH_CHAIN_SPIN_LIMIT")
    good = hip.Gemma(ctx, cfg, w)
    monkeypatch.setenv("KSEARCH_DECODE_CHAIN", "0")
    ref = hip.Gemma(ctx, cfg, w)
    assert good.forward_token(5, use_graph=False) == ref.forward_token(5, use_graph=False)
    good.close()
    ref.close()


def test_decode_chain_refuses_other_widths(ctx, monkeypatch):
    monkeypatch.setenv("KSEARCH_DECODE_CHAIN", "1")
    cfg = dict(n_layers=2, hidden=512, ffn=1024, n_q=4, n_kv=1, hd=128, vocab=4096, max_seq=64, eps=1e-6, softcap=30.0,
               rope_theta=10000.0, attn_scale=1.0)
    w = synth.gemma_weights(cfg, 911, oracle.quantize_q4k, synth.chunked(oracle.quantize_q6k), std=0.05)
    with pytest.raises(hip.KshError, match="KSEARCH_DECODE_CHAIN"):
        hip.Gemma(ctx, cfg, w)
