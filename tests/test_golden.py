"""The committed fixtures (tests/golden/small.npz): the oracle must keep
reproducing them bit for bit (CPU), and the HIP path must match them (GPU)."""
import os

import numpy as np
import pytest

import oracle

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "small.npz"))


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def test_oracle_reproduces_fixtures():
    assert np.array_equal(bits(oracle.dequant(oracle.Q4K, G["q4k_blocks"], 8 * 256)), bits(G["q4k_deq"]))
    assert np.array_equal(bits(oracle.dequant(oracle.Q6K, G["q6k_blocks"], 6 * 256)), bits(G["q6k_deq"]))
    assert np.array_equal(bits(oracle.dequant(oracle.Q40, G["q40_blocks"], 24 * 32)), bits(G["q40_deq"]))
    x = G["gemv_x"]
    assert np.array_equal(bits(oracle.matvec(oracle.Q4K, G["gemv_q4k_w"], 8, 512, x)), bits(G["gemv_q4k_y"]))
    assert np.array_equal(bits(oracle.matvec(oracle.Q6K, G["gemv_q6k_w"], 8, 512, x)), bits(G["gemv_q6k_y"]))
    out = oracle.sdpa(G["attn_q"], G["attn_k"], G["attn_v"], 2, 1, 64, 40, 0, 0.125)
    assert np.allclose(out, G["attn_out"], rtol=1e-6, atol=1e-7)       # expf may differ in the last bit across libm builds
    assert np.allclose(oracle.rope_table(8, 64, 10000.0)[7], G["rope_row_pos7_hd64"], rtol=0, atol=1e-7)
    assert np.array_equal(oracle.pack_q40(G["pack_src"]), G["pack_q40"])
    assert np.array_equal(oracle.quantize_q4k(G["quant_src"]), G["quant_q4k"])
    assert np.array_equal(oracle.quantize_q6k(G["quant_src"]), G["quant_q6k"])
    assert oracle.softcap_argmax(G["argmax_x"], 30.0) == int(G["argmax_idx"][0])


@pytest.mark.gpu
def test_hip_matches_fixtures():
    from ksearch_amd import hip
    from ksearch_amd.hip import DType

    ctx, eng = hip.Context(), hip.Eng()
    try:
        for dt, name, n in ((DType.Q4K, "q4k", 8 * 256), (DType.Q6K, "q6k", 6 * 256), (DType.Q40, "q40", 24 * 32)):
            dst = ctx.buffer_empty_f32(n)
            eng.dequant(ctx, dt, n, ctx.buffer_bytes(G[name + "_blocks"]), dst)
            assert np.array_equal(bits(ctx.read_f32(dst, n)), bits(G[name + "_deq"])), name
        bx, by = ctx.buffer_f32(G["gemv_x"]), ctx.buffer_empty_f32(8)
        for dt, name in ((DType.Q4K, "q4k"), (DType.Q6K, "q6k")):
            eng.matvec_wd(ctx, 8, 512, dt, ctx.buffer_bytes(G[f"gemv_{name}_w"]), bx, by)
            want = G[f"gemv_{name}_y"]
            assert np.abs(ctx.read_f32(by, 8) - want).max() <= 1e-3 * np.abs(want).max()
        out = ctx.buffer_empty_f32(128)
        eng.sdpa_naive_kv(ctx, 2, 1, 64, 40, DType.Q40, ctx.buffer_f32(G["attn_q"]), ctx.buffer_bytes(G["attn_k"]),
                          ctx.buffer_bytes(G["attn_v"]), ctx.buffer_f32([40, 0, 0, 0]), out, 0.125)
        assert np.abs(ctx.read_f32(out, 128) - G["attn_out"]).max() <= 1e-3 * np.abs(G["attn_out"]).max()
        dst = ctx.buffer_empty_bytes(G["pack_q40"].size)
        eng.quantize_q40(ctx, G["pack_src"].size, ctx.buffer_f32(G["pack_src"]), dst)
        assert np.array_equal(ctx.read_bytes(dst, G["pack_q40"].size), G["pack_q40"])
        for dt, name in ((DType.Q4K, "quant_q4k"), (DType.Q6K, "quant_q6k")):
            dst = ctx.buffer_empty_bytes(G[name].size)
            eng.quantize_k(ctx, dt, 512, ctx.buffer_f32(G["quant_src"]), dst)
            assert np.array_equal(ctx.read_bytes(dst, G[name].size), G[name]), name
        bi = ctx.buffer_empty_f32(1)
        eng.softcap_argmax(ctx, 1000, 30.0, ctx.buffer_f32(G["argmax_x"]), bi)
        assert int(ctx.read_f32(bi, 1)[0]) == int(G["argmax_idx"][0])
    finally:
        ctx.close()


G4 = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gemma4_small.npz"))


def _g4_model_inputs():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    from ksearch_amd import synth
    return dict(synth.GEMMA4_TINY), mg.gemma4_tiny_weights()


def test_oracle_reproduces_gemma4_fixtures():
    assert np.array_equal(bits(oracle.dequant(oracle.Q5K, G4["q5k_blocks"], 6 * 256)), bits(G4["q5k_deq"]))
    x, w = G4["ph_x"], G4["ph_w"]
    assert np.array_equal(bits(oracle.rmsnorm_per_head(x, w, 3, 128, 1e-6)), bits(G4["ph_norm"]))
    assert np.array_equal(bits(oracle.rmsnorm_per_head(x, w, 3, 128, 1e-6, G4["ph_rope"])), bits(G4["ph_rope_out"]))
    got = oracle.matvec_gelu_mul(oracle.Q4K, G4["gm_w"], 16, 512, G4["gm_x"], G4["gm_ctx"])
    assert np.allclose(got, G4["gm_y"], rtol=1e-6, atol=1e-7)                        # tanhf may differ in the last bit across libm builds
    cfg, w4 = _g4_model_inputs()
    m = oracle.Gemma4(cfg, w4)
    assert [m.kv_source(l) for l in range(cfg["n_layers"])] == list(G4["g4_kv_source"])
    for i, t in enumerate(G4["g4_prompt"]):
        tok, lg = m.forward(int(t), return_logits=True)
        assert abs(float(lg.max()) - float(G4["g4_top_logit"][i])) <= 1e-4 * abs(float(G4["g4_top_logit"][i])), i
        assert tok == int(G4["g4_tokens"][i]) or G4["g4_margin"][i] < 1e-4, i
    assert np.allclose(m.hidden(), G4["g4_hidden"], rtol=1e-4, atol=1e-5)
    m.close()


@pytest.mark.gpu
def test_hip_matches_gemma4_fixtures():
    from ksearch_amd import hip
    from ksearch_amd.hip import DType

    ctx, eng = hip.Context(), hip.Eng()
    try:
        dst = ctx.buffer_empty_f32(6 * 256)
        eng.dequant(ctx, DType.Q5K, 6 * 256, ctx.buffer_bytes(G4["q5k_blocks"]), dst)
        assert np.array_equal(bits(ctx.read_f32(dst, 6 * 256)), bits(G4["q5k_deq"]))
        bx, bw, y = ctx.buffer_f32(G4["ph_x"]), ctx.buffer_f32(G4["ph_w"]), ctx.buffer_empty_f32(3 * 128)
        eng.rmsnorm_per_head(ctx, 3, 128, 1e-6, bx, bw, y)
        assert np.abs(ctx.read_f32(y, 384) - G4["ph_norm"]).max() <= 1e-5 * np.abs(G4["ph_norm"]).max()
        eng.rmsnorm_per_head_rope_off(ctx, 3, 128, 1e-6, bx, bw, ctx.buffer_f32(G4["ph_rope"]), 0, y)
        assert np.abs(ctx.read_f32(y, 384) - G4["ph_rope_out"]).max() <= 1e-5 * np.abs(G4["ph_rope_out"]).max()
        u = ctx.buffer_empty_f32(16)
        eng.matvec_gelu_mul_at(ctx, 16, 512, DType.Q4K, ctx.buffer_bytes(G4["gm_w"]), ctx.buffer_f32(G4["gm_x"]), ctx.buffer_f32(G4["gm_ctx"]), 0, u)
        assert np.abs(ctx.read_f32(u, 16) - G4["gm_y"]).max() <= 1e-3 * np.abs(G4["gm_y"]).max()
        cfg, w4 = _g4_model_inputs()
        m = hip.Gemma4(ctx, cfg, w4)
        # teacher-forced, caches not synchronised: a Q4_0 code on a rounding boundary may differ from the oracle's
        # and stays in, so the bar on the top logit is 2e-2 here (1e-3 with synchronised caches, tests/test_gpu_gemma4.py)
        for i, t in enumerate(G4["g4_prompt"]):
            tok = m.forward_token(int(t), use_graph=True)
            top = float(m.logits().max())
            assert abs(top - float(G4["g4_top_logit"][i])) <= 2e-2 * abs(float(G4["g4_top_logit"][i])), i
            assert tok == int(G4["g4_tokens"][i]) or G4["g4_margin"][i] < 5e-2, i
        m.close()
    finally:
        ctx.close()
