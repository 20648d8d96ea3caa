"""Device quantizers and the greedy decode loop vs the CPU oracle, on a
scaled-down Gemma-shaped model (same op sequence as the full configuration)."""
import numpy as np
import pytest

import oracle
from ksearch_amd import hip, synth
from ksearch_amd.hip import DType
from tests.gpu_util import assert_close

pytestmark = pytest.mark.gpu

SMALL = dict(n_layers=3, hidden=512, ffn=1024, n_q=4, n_kv=1, hd=128, vocab=4096, max_seq=256,
             eps=1e-6, softcap=30.0, rope_theta=10000.0, attn_scale=1.0 / np.sqrt(128.0))


@pytest.fixture(scope="module")
def ctx():
    c = hip.Context()
    yield c
    c.close()


@pytest.fixture(scope="module")
def eng():
    return hip.Eng()


def test_quantize_q4k_matches_host_routine_bytes(ctx, eng):
    # weights-like signal, the reference unit test's signal, a zero and a constant block
    i = np.arange(1024, dtype=np.float32)
    sig = (np.sin(i * np.float32(0.017) + np.float32(0.3)) * np.float32(1.7)
           + np.cos(i * np.float32(0.041)) * np.float32(0.4) - np.float32(0.15)).astype(np.float32)
    sig[256:512] = 0.0
    sig[512:768] = -0.25
    x = np.concatenate([sig, synth.normal_f32(256 * 300, 400, std=0.02), synth.normal_f32(256 * 20, 401, std=3.0)])
    dst = ctx.buffer_empty_bytes(x.size // 256 * 144)
    eng.quantize_k(ctx, DType.Q4K, x.size, ctx.buffer_f32(x), dst)
    got, want = ctx.read_bytes(dst, x.size // 256 * 144), oracle.quantize_q4k(x)
    assert np.array_equal(got, want)
    back = oracle.dequant(oracle.Q4K, got, x.size)
    assert np.all(back[256:512] == 0.0) and np.abs(back[:1024] - sig).max() < 0.35


def test_quantize_q6k_matches_host_routine_bytes(ctx, eng):
    x = np.concatenate([synth.normal_f32(256 * 200, 402, std=0.02), np.zeros(256, np.float32),
                        synth.normal_f32(256 * 10, 403, std=5.0)])
    dst = ctx.buffer_empty_bytes(x.size // 256 * 210)
    eng.quantize_k(ctx, DType.Q6K, x.size, ctx.buffer_f32(x), dst)
    got, want = ctx.read_bytes(dst, x.size // 256 * 210), oracle.quantize_q6k(x)
    assert np.array_equal(got, want)


@pytest.fixture(scope="module", params=["short_context_form", "crosses_to_long_form_at_20"])
def small_model(ctx, request):
    """The decode loop has two forms of the attention / o-projection pair and switches between them by position
    (KSEARCH_SHORT_CONTEXT, read when the model is built): once with every position on the short form, once with
    the switch inside the test sequences."""
    import os
    if request.param != "short_context_form":
        os.environ["KSEARCH_SHORT_CONTEXT"] = "20"
    w = synth.gemma_weights(SMALL, 500, oracle.quantize_q4k, synth.chunked(oracle.quantize_q6k), std=0.05)
    # norm weights away from 1 so that a swapped or dropped norm shows
    rng = np.random.default_rng(501)
    for lw in w["layers"]:
        for name in ("attn_norm", "q_norm", "k_norm", "post_attn_norm", "ffn_norm", "post_ffw_norm"):
            lw[name] = (1.0 + 0.2 * rng.standard_normal(lw[name].size)).astype(np.float32)
    w["output_norm"] = (1.0 + 0.2 * rng.standard_normal(SMALL["hidden"])).astype(np.float32)
    try:
        gpu = hip.Gemma(ctx, SMALL, w)
    finally:
        os.environ.pop("KSEARCH_SHORT_CONTEXT", None)
    cpu = oracle.Gemma(SMALL, w)
    yield gpu, cpu, w
    gpu.close()
    cpu.close()


def test_forward_token_matches_oracle_teacher_forced(small_model):
    """Teacher-forced with the oracle in lockstep: a K/V value that sits on a Q4_0 rounding boundary may take the
    neighbouring code on two correct f32 implementations, so the oracle packs its own row per layer, checks that
    the device's is within one code step and continues with the device's (`adopt_rows`): every step is compared."""
    gpu, cpu, _ = small_model
    ctx = gpu.ctx
    gpu.reset()
    cpu.reset()
    rng = np.random.default_rng(502)
    toks = rng.integers(0, SMALL["vocab"], 40)
    row = SMALL["n_kv"] * SMALL["hd"] // 32 * 18
    bufs = [[hip.Buffer(ctx, hip.lib().ksh_gemma_kv(gpu.h, l, w), owned=False) for w in (0, 1)]
            for l in range(SMALL["n_layers"])]
    agree, flipped = 0, 0
    for i, t in enumerate(toks):
        g_next = gpu.forward_token(int(t), use_graph=False)
        rows = np.stack([np.stack([ctx.read_bytes(bufs[l][w], row, i * row) for w in (0, 1)]) for l in range(SMALL["n_layers"])])
        c_next, c_logits = cpu.forward(int(t), return_logits=True, adopt_rows=rows)
        assert cpu.row_max_step.max() <= 1.0 + 1e-3, (i, cpu.row_max_step)      # a flip is one code step, never more
        flipped += int(cpu.row_diff_bytes.sum())
        g_logits = gpu.logits()
        # the device argmax follows the oracle's rule on the device's own logits
        assert g_next == oracle.softcap_argmax(g_logits, SMALL["softcap"])
        assert_close(g_logits, c_logits, 1e-3, f"logits at step {i}")
        assert_close(gpu.hidden(), cpu.hidden(), 1e-3, f"hidden at step {i}")
        top2 = np.sort(c_logits)[-2:]
        if top2[1] - top2[0] > 2e-3 * max(abs(top2[1]), float(np.sqrt(np.mean(c_logits ** 2)))):
            assert g_next == c_next, f"step {i}: margin {top2[1] - top2[0]}"
            agree += 1
    print(f"small model, 40 teacher-forced steps: {flipped} of {40 * SMALL['n_layers'] * 2 * row} KV bytes differ by one code")
    # (measured: 1 - 2 of 17,280 bytes; the bound is 34)
    assert agree >= 30 and flipped <= 0.002 * 40 * SMALL["n_layers"] * 2 * row and gpu.pos == cpu.pos == len(toks)
    with pytest.raises(hip.KshError, match="outside the vocabulary"):
        gpu.forward_token(SMALL["vocab"])


def test_generate_graph_equals_eager_and_oracle(small_model):
    gpu, cpu, _ = small_model
    rng = np.random.default_rng(503)
    prompt = [int(t) for t in rng.integers(0, SMALL["vocab"], 12)]
    n_new = 48
    gpu.reset()
    eager, _, _ = gpu.generate(prompt, n_new, use_graph=False)
    gpu.reset()
    graph, _, ms = gpu.generate(prompt, n_new, use_graph=True)
    assert graph == eager                     # same kernels, same order: bit-identical
    gpu.reset()
    assert gpu.generate(prompt, n_new, use_graph=True)[0] == graph      # replay after reset
    assert gpu.launches_per_token > 0
    # the oracle's greedy continuation
    cpu.reset()
    for t in prompt[:-1]:
        cpu.forward(t, want_logits=False)
    want, margins, t = [], [], prompt[-1]
    for _ in range(n_new):
        t, lg = cpu.forward(t, return_logits=True)
        s = np.sort(lg)
        margins.append(float((s[-1] - s[-2]) / max(abs(s[-1]), float(np.sqrt(np.mean(lg ** 2))))))
        want.append(t)
    # identical until (if ever) the oracle's own top-2 margin drops under the numeric tolerance
    n_same = next((i for i, (a, b) in enumerate(zip(graph, want)) if a != b), n_new)
    assert n_same == n_new or margins[n_same] < 1e-3, (n_same, margins[n_same] if n_same < n_new else None)
    assert n_same >= 8


def test_profile_mode_prints_sections_and_changes_nothing(ctx, capfd, monkeypatch):
    """KSEARCH_PROFILE (gemma_prim.rs:885, 1260-1273): every step prints one line with its per-section times; the
    tokens are those of the unprofiled model."""
    w = synth.gemma_weights(SMALL, 500, oracle.quantize_q4k, synth.chunked(oracle.quantize_q6k), std=0.05)
    prompt = [int(t) for t in np.random.default_rng(505).integers(0, SMALL["vocab"], 5)]
    plain = hip.Gemma(ctx, SMALL, w)
    want, _, _ = plain.generate(prompt, 6, use_graph=True)
    plain.close()
    monkeypatch.setenv("KSEARCH_PROFILE", "1")
    prof = hip.Gemma(ctx, SMALL, w)
    monkeypatch.delenv("KSEARCH_PROFILE")
    capfd.readouterr()
    got, _, _ = prof.generate(prompt, 6, use_graph=True, serial_prefill=True)
    prof.close()
    err = capfd.readouterr().err
    assert got == want
    lines = [l for l in err.splitlines() if l.startswith("[profile]")]
    assert len([l for l in lines if " decode " in l]) == 6 and len([l for l in lines if " prefill " in l]) == len(prompt) - 1
    fields = dict(f.split("=") for f in lines[-1].split()[2:])
    assert set(fields) == {"pos", "embed", "prepass", "attn", "mlp", "ple", "logits+sync", "total"}
    ms = {k: float(v[:-2]) for k, v in fields.items() if k != "pos"}
    assert ms["attn"] > 0 and ms["mlp"] > 0 and ms["logits+sync"] > 0
    assert abs(ms["total"] - sum(v for k, v in ms.items() if k != "total")) < 1e-2


def test_generate_refuses_past_max_seq(small_model):
    gpu, _, _ = small_model
    gpu.reset()
    with pytest.raises(hip.KshError, match="max_seq exceeded"):
        gpu.generate([1, 2, 3], SMALL["max_seq"], use_graph=False)


def test_plans_are_warmed_at_load_and_picked_up(ctx, tmp_path, monkeypatch):
    """GemmaPrimModel's load warms the schedule search for its GEMV shapes (gemma_prim.rs:254-290) unless
    KSEARCH_SKIP_BEAM is set: the model's kinds leave plan files, a second model is served from them, and the
    decode step under the planned schedules still matches the oracle."""
    monkeypatch.setenv("KSEARCH_BEAM_CACHE", str(tmp_path / "beam"))
    monkeypatch.delenv("KSEARCH_SKIP_BEAM", raising=False)
    w = synth.gemma_weights(SMALL, 500, oracle.quantize_q4k, synth.chunked(oracle.quantize_q6k), std=0.05)
    gpu = hip.Gemma(ctx, SMALL, w)
    names = sorted(f.name.split("_0")[0].rsplit("_", 1)[0] for f in (tmp_path / "beam").glob("*.txt"))
    kinds = {n.split("_" + str(SMALL["hidden"]))[0] for n in names}
    assert any(n.startswith("rms_matvec_qkv_q4k") for n in names) and any(n.startswith("rms_matvec_gate_up_q4k") for n in names)
    assert any(n.startswith("matvec_q4k") for n in names) and any(n.startswith("attend_decode_q40") for n in names), names
    stamp = {f.name: f.stat().st_mtime_ns for f in (tmp_path / "beam").glob("*.txt")}
    cpu = oracle.Gemma(SMALL, w)
    row = SMALL["n_kv"] * SMALL["hd"] // 32 * 18
    bufs = [[hip.Buffer(ctx, hip.lib().ksh_gemma_kv(gpu.h, l, x), owned=False) for x in (0, 1)] for l in range(SMALL["n_layers"])]
    for i, t in enumerate(np.random.default_rng(504).integers(0, SMALL["vocab"], 6)):
        gpu.forward_token(int(t), use_graph=bool(i & 1))
        rows = np.stack([np.stack([ctx.read_bytes(bufs[l][x], row, i * row) for x in (0, 1)]) for l in range(SMALL["n_layers"])])
        _, c_logits = cpu.forward(int(t), return_logits=True, adopt_rows=rows)
        assert cpu.row_max_step.max() <= 1.0 + 1e-3
        assert_close(gpu.logits(), c_logits, 1e-3, f"logits at step {i} under planned schedules")
    gpu.close()
    again = hip.Gemma(ctx, SMALL, w)                       # every search is served from its file: none is rewritten
    assert {f.name: f.stat().st_mtime_ns for f in (tmp_path / "beam").glob("*.txt")} == stamp
    again.close()
    cpu.close()
    del kinds
