"""Batched prefill: the row / batch forms of the kinds a prompt chunk is made of, each against the serial oracle op
applied token by token (the reference's own check is batch-versus-serial, crates/ksearch_kernels/examples/
check_mul_mm.rs:134-247), and the chunked prompt pass of the decode loop against the oracle in lockstep."""
import numpy as np
import pytest

import oracle
from ksearch_amd import hip, synth
from ksearch_amd.hip import DType, Kind
from tests.gpu_util import assert_close, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = hip.Context()
    yield c
    c.close()


def run1(ctx, kind, dims, dtypes, params, ins, outs):
    k = ctx.compile(hip.make_desc(kind, dims, dtypes, params))
    ctx.encode_multi(k, ins, outs)
    ctx.synchronize()
    return k


def test_rmsnorm_rows_forms(ctx):
    rng = np.random.default_rng(700)
    n, rows, eps = 512, 37, 1e-6
    x = rng.standard_normal((rows, n)).astype(np.float32) * 3
    res = rng.standard_normal((rows, n)).astype(np.float32)
    w = (1 + 0.2 * rng.standard_normal(n)).astype(np.float32)
    w2 = (1 + 0.2 * rng.standard_normal(n)).astype(np.float32)
    bx, br, bw, bw2 = ctx.buffer_f32(x), ctx.buffer_f32(res), ctx.buffer_f32(w), ctx.buffer_f32(w2)
    by, by2 = ctx.buffer_empty_f32(rows * n), ctx.buffer_empty_f32(rows * n)
    # plain, with residual, with residual and scale: bit-identical to the single-row op row by row
    for has_res, scale in ((0, None), (1, None), (1, 0.75)):
        run1(ctx, Kind.RMSNORM, (n, has_res, int(scale is not None), rows), (), (eps, scale or 0.0),
             [bx, bw] + ([br] if has_res else []), [by])
        got = ctx.read_f32(by, rows * n).reshape(rows, n)
        for r in range(rows):
            want = oracle.rmsnorm(x[r], w, eps, res[r] if has_res else None, scale)
            assert_close(got[r], want, 1e-5, f"rmsnorm rows {has_res} {scale} row {r}")
    run1(ctx, Kind.RMSNORM_ADD_THEN_RMSNORM, (n, rows), (), (eps,), [bx, bw, br, bw2], [by, by2])
    g1, g2 = ctx.read_f32(by, rows * n).reshape(rows, n), ctx.read_f32(by2, rows * n).reshape(rows, n)
    for r in range(rows):
        w1, w2_ = oracle.rmsnorm_add_then_rmsnorm(x[r], w, res[r], w2, eps)
        assert_close(g1[r], w1, 1e-5, "add_then x")
        assert_close(g2[r], w2_, 1e-5, "add_then x2")
    # in place on the residual stream, as the chunk pass uses it
    run1(ctx, Kind.RMSNORM, (n, 1, 0, rows), (), (eps,), [bx, bw, br], [br])
    got = ctx.read_f32(br, rows * n).reshape(rows, n)
    for r in range(rows):
        assert_close(got[r], oracle.rmsnorm(x[r], w, eps, res[r]), 1e-5, "in place")


def test_gather_batch_and_gelu_rows(ctx):
    rng = np.random.default_rng(701)
    n, vocab, t = 512, 300, 19
    table = synth.q6k_blocks(vocab * n // 256, 702)
    ids = rng.integers(0, vocab, t)
    bt, bi, bo = ctx.buffer_bytes(table), ctx.buffer_f32(ids.astype(np.float32)), ctx.buffer_empty_f32(t * n)
    run1(ctx, Kind.COPY_SCALE_INDEXED, (n, vocab, t), (DType.Q6K,), (1.5,), [bt, bi], [bo])
    got = ctx.read_f32(bo, t * n).reshape(t, n)
    for i, tok in enumerate(ids):
        want = oracle.copy_scale_indexed(oracle.Q6K, table, int(tok), n, 1.5)
        assert np.array_equal(got[i].view(np.uint32), want.view(np.uint32)), i


@pytest.mark.parametrize("hd,n_q,n_kv", [(128, 4, 1), (256, 8, 1), (256, 4, 2)])
def test_per_head_qkv_q40_batch(ctx, hd, n_q, n_kv):
    rng = np.random.default_rng(703)
    t, max_seq, pos0, eps = 11, 64, 9, 1e-6
    q = rng.standard_normal((t, n_q * hd)).astype(np.float32)
    k = rng.standard_normal((t, n_kv * hd)).astype(np.float32)
    v = rng.standard_normal((t, n_kv * hd)).astype(np.float32)
    qw, kw = (1 + 0.2 * rng.standard_normal(hd)).astype(np.float32), (1 + 0.2 * rng.standard_normal(hd)).astype(np.float32)
    rope = oracle.rope_table(max_seq, hd, 10000.0)
    row = n_kv * hd // 32 * 18
    meta = np.array([pos0 + 1, 0, 0, pos0], np.float32)
    bq, bk, bv = ctx.buffer_f32(q), ctx.buffer_f32(k), ctx.buffer_f32(v)
    kc, vc = ctx.buffer_bytes(np.zeros(max_seq * row, np.uint8)), ctx.buffer_bytes(np.zeros(max_seq * row, np.uint8))
    run1(ctx, Kind.RMSNORM_PER_HEAD_QKV_Q40, (n_q, n_kv, hd, max_seq, t), (), (eps,),
         [bq, ctx.buffer_f32(qw), ctx.buffer_f32(rope), bk, ctx.buffer_f32(kw), bv, ctx.buffer_f32(meta)], [bq, kc, vc])
    gq = ctx.read_f32(bq, t * n_q * hd).reshape(t, -1)
    gk, gv = ctx.read_bytes(kc, max_seq * row).reshape(max_seq, row), ctx.read_bytes(vc, max_seq * row).reshape(max_seq, row)
    for i in range(t):
        wq_, wk_, wv_ = oracle.rmsnorm_per_head_qkv_q40(q[i], qw, rope[pos0 + i], k[i], kw, v[i], n_q, n_kv, hd, eps)
        assert_close(gq[i], wq_, 1e-5, f"q token {i}")
        # packed rows: identical, or one code apart where a value sits on a rounding boundary
        for got, want in ((gk[pos0 + i], wk_), (gv[pos0 + i], wv_)):
            if not np.array_equal(got, want):
                dg, dw = oracle.dequant(oracle.Q40, got, n_kv * hd), oracle.dequant(oracle.Q40, want, n_kv * hd)
                assert np.abs(dg - dw).max() <= np.abs(dw).max() / 7 * 1.01 and (got != want).sum() <= 2
    assert not gk[:pos0].any() and not gk[pos0 + t:].any() and not gv[:pos0].any() and not gv[pos0 + t:].any()


@pytest.mark.parametrize("hd,n_q,n_kv,sched", [(256, 8, 1, None), (128, 4, 1, None), (256, 4, 2, None), (64, 4, 2, None),
                                               (256, 8, 1, dict(vec=1)), (256, 8, 1, dict(vec=2)), (256, 4, 2, dict(vec=2)),
                                               (256, 8, 1, dict(vec=3)), (256, 4, 2, dict(k_split=3)), (512, 8, 1, None), (512, 4, 2, dict(k_split=2))])
@pytest.mark.parametrize("t,pos0,window", [(5, 0, 1 << 20), (33, 100, 1 << 20), (40, 150, 64), (130, 3, 1 << 20), (17, 290, 1 << 20)])
def test_sdpa_batch_equals_the_serial_oracle(ctx, hd, n_q, n_kv, sched, t, pos0, window):
    """Token i of the chunk attends rows [start_i, pos0 + i] of the one cache: the same numbers as the single-token
    oracle attention with that range -- register form (vec=3; the default up to 16 tokens), tile form (vec=1 or other
    head sizes), matrix-core forms (heads of 256 and 512: the default from 17 tokens on, one or several partitions per
    token in workgroups of their own, heads of 512 as two workgroups with half of the V dimensions each; vec=2 with
    up to 64 tokens of 256-wide heads deals the partitions by length), with and without a sliding window."""
    max_t = 320
    row = n_kv * hd // 32 * 18
    kk, vv = synth.q40_blocks(max_t * n_kv * hd // 32, 710), synth.q40_blocks(max_t * n_kv * hd // 32, 711)
    q = synth.normal_f32(t * n_q * hd, 712).reshape(t, -1)
    scale = 1.0 / np.sqrt(hd)
    k = ctx.compile(hip.make_desc(Kind.SDPA_BATCH, (n_q, n_kv, hd, max_t, t, 0), (DType.Q40, DType.F32), (scale,), sched))
    vec = (sched or {}).get("vec", 0)
    assert ("mfma" in k.name) == (vec == 2 or (vec == 0 and hd in (256, 512) and t > 16)), k.name
    nwg = k.info.sched.k_split
    if sched and sched.get("k_split"):
        assert nwg == sched["k_split"]
    elif "mfma" in k.name and vec == 0:
        assert nwg == 1          # the default of the one-workgroup-per-token form
    tmp, out = ctx.buffer_empty_f32(t * n_q * nwg * (hd + 2)), ctx.buffer_empty_f32(t * n_q * hd)
    meta = np.array([pos0 + 1, 0, window, 0], np.float32)
    ctx.encode_multi(k, [ctx.buffer_f32(q), ctx.buffer_bytes(kk), ctx.buffer_bytes(vv), ctx.buffer_f32(meta)], [tmp, out])
    ctx.synchronize()
    got = ctx.read_f32(out, t * n_q * hd).reshape(t, -1)
    for i in range(t):
        tlen = min(pos0 + 1 + i, window)
        start = pos0 + 1 + i - tlen
        want = oracle.sdpa(q[i], kk, vv, n_q, n_kv, hd, tlen, start, scale)
        assert_close(got[i], want, 1e-3, f"{k.name} token {i} rows [{start}, {start + tlen})")
    del row


@pytest.mark.parametrize("wdt,batch,sched", [(DType.Q4K, 45, None), (DType.Q6K, 45, None), (DType.Q4K, 5, None), (DType.Q4K, 32, None),
                                             (DType.Q4K, 64, None), (DType.Q4K, 45, dict(nr0=128)), (DType.Q4K, 100, None)])
def test_mul_mm_f32_activations(ctx, wdt, batch, sched):
    """f32 activations go through as hi + lo f16 parts: the result keeps the GEMV's accuracy (1e-5 of the float64
    product), where a single f16 rounding of x would leave 3e-4.  Up to 64 tokens over Q4_K weights take the
    small-batch form (32 weight rows per workgroup, K split over its waves) unless the schedule asks for the
    128 x 128 tile; both forms, one and two token tiles, a ragged last row tile."""
    rows, cols = 400, 2048
    w = synth.q4k_blocks(rows * cols // 256, 720) if wdt == DType.Q4K else synth.q6k_blocks(rows * cols // 256, 720)
    x = synth.normal_f32(batch * cols, 721).reshape(batch, cols)
    x[3] *= 1e-3           # small rows: the low part is kept 2^11 up, so it stays a normal f16
    x[4] *= 300.0
    k = ctx.compile(hip.make_desc(Kind.MATVEC_BATCH, (rows, cols, batch), (wdt, DType.F32, DType.F32), (), sched))
    assert ("skinny" in k.name) == (wdt == DType.Q4K and batch <= 64 and sched is None), k.name
    by = ctx.buffer_empty_f32(batch * rows)
    ctx.encode_multi(k, [ctx.buffer_bytes(w), ctx.buffer_f32(x)], [by])
    ctx.synchronize()
    got = ctx.read_f32(by, batch * rows).reshape(batch, rows)
    odt = oracle.Q4K if wdt == DType.Q4K else oracle.Q6K
    worst = 0.0
    for t in range(batch):
        want = oracle.matvec_f64(odt, w, rows, cols, x[t])
        worst = max(worst, float(rel_err(got[t], want).max()))
    assert worst <= 2e-5, worst


SMALL = dict(n_layers=3, hidden=512, ffn=1024, n_q=4, n_kv=1, hd=128, vocab=4096, max_seq=400,
             eps=1e-6, softcap=30.0, rope_theta=10000.0, attn_scale=1.0 / np.sqrt(128.0))


@pytest.fixture(scope="module")
def small_model(ctx):
    w = synth.gemma_weights(SMALL, 730, oracle.quantize_q4k, synth.chunked(oracle.quantize_q6k), std=0.05)
    rng = np.random.default_rng(731)
    for lw in w["layers"]:
        for name in ("attn_norm", "q_norm", "k_norm", "post_attn_norm", "ffn_norm", "post_ffw_norm"):
            lw[name] = (1.0 + 0.2 * rng.standard_normal(lw[name].size)).astype(np.float32)
    w["output_norm"] = (1.0 + 0.2 * rng.standard_normal(SMALL["hidden"])).astype(np.float32)
    gpu, cpu = hip.Gemma(ctx, SMALL, w), oracle.Gemma(SMALL, w)
    yield gpu, cpu
    gpu.close()
    cpu.close()


def lockstep_prompt(ctx, gpu, cpu, cfg, toks, first_pos=0):
    """After the device has prefilled `toks` from position `first_pos`: the oracle walks the same positions, packing
    its own K / V rows, checking the device's against them (one code step at most) and adopting them."""
    n_layers, row = cfg["n_layers"], cfg["n_kv"] * cfg["hd"] // 32 * 18
    n = len(toks)
    kv = np.stack([np.stack([gpu.kv(l, w, (first_pos + n) * row)[first_pos * row:].reshape(n, row) for w in (0, 1)])
                   for l in range(n_layers)])                      # [layer, which, pos, row]
    flipped = 0
    for i, t in enumerate(toks):
        cpu.forward(int(t), want_logits=False, adopt_rows=np.ascontiguousarray(kv[:, :, i]))
        assert cpu.row_max_step.max() <= 1.0 + 1e-3, (i, cpu.row_max_step)
        flipped += int(cpu.row_diff_bytes.sum())
    assert flipped <= 0.02 * n * n_layers * 2 * row, flipped
    return flipped


@pytest.mark.parametrize("n_prompt", [2, 31, 64, 300])
def test_prefill_chunk_matches_oracle_in_lockstep(ctx, small_model, n_prompt):
    """prefill_chunk(N tokens) leaves the KV rows of N decode steps (up to one-code flips) and the next decode step
    gives the oracle's logits; 300 tokens cross the oracle's 128-row switch to split-KV attention."""
    gpu, cpu = small_model
    toks = np.random.default_rng(740 + n_prompt).integers(0, SMALL["vocab"], n_prompt + 3)
    gpu.reset()
    cpu.reset()
    gpu.prefill_chunk(toks[:n_prompt])
    assert gpu.pos == n_prompt
    lockstep_prompt(ctx, gpu, cpu, SMALL, toks[:n_prompt])
    row = SMALL["hd"] // 32 * 18
    bufs = [[hip.Buffer(ctx, hip.lib().ksh_gemma_kv(gpu.h, l, w), owned=False) for w in (0, 1)] for l in range(SMALL["n_layers"])]
    for i in range(n_prompt, n_prompt + 3):          # decode steps behind the chunk, graph and eager
        g_next = gpu.forward_token(int(toks[i]), use_graph=bool(i & 1))
        rows = np.stack([np.stack([ctx.read_bytes(bufs[l][w], row, i * row) for w in (0, 1)]) for l in range(SMALL["n_layers"])])
        c_next, c_logits = cpu.forward(int(toks[i]), return_logits=True, adopt_rows=rows)
        assert cpu.row_max_step.max() <= 1.0 + 1e-3
        assert_close(gpu.logits(), c_logits, 1e-3, f"logits at position {i}")
        top2 = np.sort(c_logits)[-2:]
        if top2[1] - top2[0] > 2e-3 * max(abs(top2[1]), float(np.sqrt(np.mean(c_logits ** 2)))):
            assert g_next == c_next


def test_prefill_long_prompt_takes_two_chunks(ctx):
    """1100 prompt tokens are a chunk of 1024 and one of 76 (heads of 256: both chunks' attention on the matrix cores,
    the second over the first one's rows; GEMMs over K slices at 1024 and at 76 rows, gate | up at 1024 rows with
    256 tiles of 128 tokens, so of 64 tokens each; partial sums travelling between the GEMMs):
    every K / V row within one code step of the oracle's, which walks the positions one by one, and the decode steps
    behind the prompt at 1e-3."""
    cfg = dict(n_layers=2, hidden=512, ffn=2048, n_q=4, n_kv=1, hd=256, vocab=4096, max_seq=1200,
               eps=1e-6, softcap=30.0, rope_theta=10000.0, attn_scale=1.0 / 16.0)
    w = synth.gemma_weights(cfg, 760, oracle.quantize_q4k, synth.chunked(oracle.quantize_q6k), std=0.05)
    gpu, cpu = hip.Gemma(ctx, cfg, w), oracle.Gemma(cfg, w)
    n_prompt = 1100
    toks = np.random.default_rng(761).integers(0, cfg["vocab"], n_prompt + 2)
    gpu.prefill_chunk(toks[:n_prompt])
    assert gpu.pos == n_prompt
    lockstep_prompt(ctx, gpu, cpu, cfg, toks[:n_prompt])
    row = cfg["hd"] // 32 * 18
    bufs = [[hip.Buffer(ctx, hip.lib().ksh_gemma_kv(gpu.h, l, w_), owned=False) for w_ in (0, 1)] for l in range(cfg["n_layers"])]
    for i in range(n_prompt, n_prompt + 2):
        gpu.forward_token(int(toks[i]), use_graph=bool(i & 1))
        rows = np.stack([np.stack([ctx.read_bytes(bufs[l][w_], row, i * row) for w_ in (0, 1)]) for l in range(cfg["n_layers"])])
        _, c_logits = cpu.forward(int(toks[i]), return_logits=True, adopt_rows=rows)
        assert cpu.row_max_step.max() <= 1.0 + 1e-3
        assert_close(gpu.logits(), c_logits, 1e-3, f"logits at position {i}")
    gpu.close()
    cpu.close()


def test_prefill_in_two_calls_and_serial_prefill_agree(ctx, small_model):
    """A prompt fed as 40 + 1 + 23 tokens (a single token goes through the decode step) leaves the same cache as one
    call, and generate() gives the same continuation with batched and with token-by-token prefill unless a Q4_0 flip
    separates the two (then the first differing token sits on a margin below the tolerance of the other run)."""
    gpu, cpu = small_model
    toks = [int(t) for t in np.random.default_rng(750).integers(0, SMALL["vocab"], 64)]
    row = SMALL["hd"] // 32 * 18
    gpu.reset()
    gpu.prefill_chunk(toks)
    one = [gpu.kv(l, w, 64 * row) for l in range(3) for w in (0, 1)]
    gpu.reset()
    gpu.prefill_chunk(toks[:40])
    gpu.prefill_chunk(toks[40:41])
    gpu.prefill_chunk(toks[41:])
    assert gpu.pos == 64
    cpu.reset()
    lockstep_prompt(ctx, gpu, cpu, SMALL, toks)
    parts = [gpu.kv(l, w, 64 * row) for l in range(3) for w in (0, 1)]
    differing = sum(int((a != b).sum()) for a, b in zip(one, parts))
    assert differing <= 0.02 * 6 * 64 * row, differing
    gpu.reset()
    a, pre_a, _ = gpu.generate(toks, 16, use_graph=True)
    gpu.reset()
    b, pre_b, _ = gpu.generate(toks, 16, use_graph=True, serial_prefill=True)
    print(f"prefill of 63 tokens: batched {pre_a:.2f} ms, token by token {pre_b:.2f} ms; continuations equal for "
          f"{next((i for i, (x, y) in enumerate(zip(a, b)) if x != y), 16)} of 16 tokens")
    with pytest.raises(hip.KshError, match="max_seq exceeded"):
        gpu.prefill_chunk([1] * 400)
    with pytest.raises(hip.KshError, match="outside the vocabulary"):
        gpu.prefill_chunk([1, SMALL["vocab"]])
