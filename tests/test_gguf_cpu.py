"""GGUF reader, host dequantizers and GemmaConfig::from_gguf, through the C ABI.  No GPU work."""
import numpy as np
import pytest

import oracle
from ksearch_amd import hip, synth
from ksearch_amd.hip import GgmlType
from tests import gguf_writer as gw


def test_reader_metadata_tensors_and_alignment(tmp_path):
    rng = np.random.default_rng(700)
    a = rng.standard_normal(6 * 32).astype(np.float32)
    b = synth.q4k_blocks(3 * 2, 701)
    c = rng.integers(0, 256, 100, dtype=np.uint8).astype(np.float16)
    meta = [("general.architecture", gw.STR, "gemma4"), ("general.alignment", gw.U32, 64), ("a.u8", gw.U8, 200), ("a.i32", gw.I32, 12345),
            ("a.u64", gw.U64, 77), ("a.f32", gw.F32, 0.25), ("a.f64", gw.F64, 1e-6), ("a.bool", gw.BOOL, 1), ("a.u16", gw.U16, 513),
            ("arr.u32", gw.ARR, (gw.U32, [5, 6, 7])), ("arr.i32", gw.ARR, (gw.I32, [9, 8])), ("arr.bool", gw.ARR, (gw.BOOL, [1, 0, 1, 1])),
            ("arr.str", gw.ARR, (gw.STR, ["x", "yz", ""])), ("arr.f32", gw.ARR, (gw.F32, [1.5, 2.5])), ("arr.i8", gw.ARR, (gw.I8, [-1, 2, -3]))]
    tensors = [("t.f32", GgmlType.F32, (32, 6), a), ("t.q4k", GgmlType.Q4_K, (512, 3), b), ("t.f16", GgmlType.F16, (100,), c)]
    path = tmp_path / "m.gguf"
    data_off = gw.write(str(path), meta, tensors, alignment=64)
    assert data_off % 64 == 0
    with hip.Gguf(str(path)) as g:
        assert g.version == 3 and g.tensor_names() == ["t.f32", "t.q4k", "t.f16"]
        assert g.get_str("general.architecture") == "gemma4" and g.get_str("a.i32") is None and g.get_str("nope") is None
        assert g.get_u32("a.i32") == 12345 and g.get_u32("a.u64") == 77 and g.get_u32("a.u16") == 513
        assert g.get_u32("a.u8") is None and g.get_u32("a.f32") is None        # get_u32 takes U32 / I32 / U64 / U16 only
        assert g.get_f32("a.f32") == 0.25 and abs(g.get_f32("a.f64") - 1e-6) < 1e-12 and g.get_f32("a.i32") is None
        assert g.get_list("arr.u32") == [5, 6, 7] and g.get_list("arr.i32") == [9, 8] and g.get_list("a.i32") == [12345]
        assert g.get_list("arr.bool") == [True, False, True, True] and g.get_list("arr.str") is None and g.get_list("arr.f32") is None
        ty, dims, raw = g.tensor("t.f32")
        assert (ty, dims) == (GgmlType.F32, (32, 6)) and np.array_equal(raw.view(np.float32), a)
        ty, dims, raw = g.tensor("t.q4k")
        assert (ty, dims) == (GgmlType.Q4_K, (512, 3)) and np.array_equal(raw, b)
        ty, dims, raw = g.tensor("t.f16")
        assert dims == (100,) and np.array_equal(raw.view(np.float16), c)
        assert g.has_tensor("t.f16") and not g.has_tensor("t.f17")
        with pytest.raises(hip.KshError, match="tensor not found: t.f17"):
            g.tensor("t.f17")


def test_reader_rejects_malformed_files(tmp_path):
    p = str(tmp_path / "bad.gguf")
    t = [("t", GgmlType.F32, (8,), np.zeros(8, np.float32))]
    gw.write(p, [], t, magic=0x12345678)
    with pytest.raises(hip.KshError, match="bad magic"):
        hip.Gguf(p)
    gw.write(p, [], t, version=1)
    with pytest.raises(hip.KshError, match="unsupported GGUF version 1"):
        hip.Gguf(p)
    gw.write(p, [("k", gw.U32, 1)], t)
    whole = open(p, "rb").read()
    open(p, "wb").write(whole[:40])                      # cut inside the metadata table
    with pytest.raises(hip.KshError, match="truncated"):
        hip.Gguf(p)
    open(p, "wb").write(whole[:-8])                      # cut inside the tensor data
    with pytest.raises(hip.KshError, match="outside the file"):
        hip.Gguf(p)
    gw.write(p, [], [("t", GgmlType.Q4_K, (100,), np.zeros(144, np.uint8))])
    with pytest.raises(hip.KshError, match="not divisible by block"):
        hip.Gguf(p)
    # dims whose product overflows 64 bits
    gw.write(p, [], [("huge", GgmlType.F32, (2 ** 40, 2 ** 40), np.zeros(8, np.float32))])
    with pytest.raises(hip.KshError, match="outside the file"):
        hip.Gguf(p)
    with pytest.raises(hip.KshError, match="failed to open"):
        hip.Gguf(str(tmp_path / "missing.gguf"))
    # a type this reader does not know is refused when the tensor is asked for, not at open
    gw.write(p, [], [("odd", 10, (256,), np.zeros(84, np.uint8))] + t)
    with hip.Gguf(p) as g:
        assert g.tensor("t")[1] == (8,)
        with pytest.raises(hip.KshError, match="unsupported ggml type id 10"):
            g.tensor("odd")


def test_host_dequant_types():
    every = np.arange(65536, dtype=np.uint16)
    got = hip.gguf_dequant_host(GgmlType.F16, every.view(np.uint8), 65536)
    want = every.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))           # NaN payloads included
    assert np.array_equal(hip.gguf_dequant_host(GgmlType.BF16, every.view(np.uint8), 65536).view(np.uint32), every.astype(np.uint32) << 16)
    rng = np.random.default_rng(702)
    f = rng.standard_normal(100).astype(np.float32)
    assert np.array_equal(hip.gguf_dequant_host(GgmlType.F32, f.view(np.uint8), 100), f)
    q40 = synth.q40_blocks(40, 703)
    assert np.array_equal(hip.gguf_dequant_host(GgmlType.Q4_0, q40, 40 * 32), oracle.dequant(oracle.Q40, q40, 40 * 32))
    # Q8_0 / Q4_1 / Q5_1: closed forms of the GGML block layouts
    nb = 25
    d = rng.uniform(0.01, 0.1, nb).astype(np.float16)
    m = rng.uniform(-1, 1, nb).astype(np.float16)
    q8 = rng.integers(-128, 128, (nb, 32), dtype=np.int8)
    blk = np.concatenate([d.view(np.uint8).reshape(nb, 2), q8.view(np.uint8)], axis=1)
    assert np.array_equal(hip.gguf_dequant_host(GgmlType.Q8_0, blk, nb * 32).reshape(nb, 32), q8.astype(np.float32) * d.astype(np.float32)[:, None])
    qs = rng.integers(0, 256, (nb, 16), dtype=np.uint8)
    blk = np.concatenate([d.view(np.uint8).reshape(nb, 2), m.view(np.uint8).reshape(nb, 2), qs], axis=1)
    codes = np.concatenate([qs & 15, qs >> 4], axis=1).astype(np.float32)
    want = codes * d.astype(np.float32)[:, None] + m.astype(np.float32)[:, None]
    assert np.array_equal(hip.gguf_dequant_host(GgmlType.Q4_1, blk, nb * 32).reshape(nb, 32), want)
    qh = rng.integers(0, 2 ** 32, nb, dtype=np.uint64).astype(np.uint32)
    blk = np.concatenate([d.view(np.uint8).reshape(nb, 2), m.view(np.uint8).reshape(nb, 2), qh.view(np.uint8).reshape(nb, 4), qs], axis=1)
    bits = ((qh[:, None] >> np.arange(32, dtype=np.uint32)[None, :]) & 1).astype(np.float32)     # element j takes bit j
    want = (codes + 16 * bits) * d.astype(np.float32)[:, None] + m.astype(np.float32)[:, None]
    assert np.array_equal(hip.gguf_dequant_host(GgmlType.Q5_1, blk, nb * 32).reshape(nb, 32), want)
    with pytest.raises(hip.KshError, match="converted on the device"):
        hip.gguf_dequant_host(GgmlType.Q6_K, np.zeros(210, np.uint8), 256)


def _cfg_file(tmp_path, extra, tensors=()):
    meta = [("general.architecture", gw.STR, "gemma4"), ("gemma4.block_count", gw.U32, 12), ("gemma4.embedding_length", gw.U32, 1536),
            ("gemma4.attention.head_count", gw.U32, 8)] + extra
    p = str(tmp_path / "cfg.gguf")
    gw.write(p, meta, list(tensors) or [("x", GgmlType.F32, (8,), np.zeros(8, np.float32))])
    return p


def test_config_from_gguf_defaults_and_overrides(tmp_path):
    """crates/ksearch_gemma/src/lib.rs:39-122: the defaults, the per-layer and scalar feed-forward lengths, the
    pattern fallback (every sixth layer attends everything), vocab from the embedding table's rows."""
    with hip.Gguf(_cfg_file(tmp_path, [])) as g:
        cfg, ffn, swa = g.gemma4_config(4096)
    assert cfg["n_layers"] == 12 and cfg["hidden"] == 1536 and cfg["n_q"] == 8 and cfg["n_kv"] == 1
    assert (cfg["hd_full"], cfg["hd_swa"], cfg["sliding_window"], cfg["shared_kv_layers"]) == (512, 256, 512, 0)
    assert cfg["eps"] == np.float32(1e-6) and cfg["softcap"] == 30.0 and cfg["rope_theta_full"] == 1e6 and cfg["rope_theta_swa"] == 1e4
    assert cfg["partial_rotary"] == 0.25 and cfg["attn_scale"] == 1.0 and cfg["vocab"] == 262144 and cfg["max_seq"] == 4096
    assert cfg["ple_dim"] == 0                                   # no per-layer tables in the file
    assert ffn == [6144] * 12 and swa == [(i + 1) % 6 != 0 for i in range(12)]
    extra = [("gemma4.attention.head_count_kv", gw.ARR, (gw.U32, [2])), ("gemma4.attention.key_length", gw.U32, 256),
             ("gemma4.attention.key_length_swa", gw.U32, 128), ("gemma4.attention.sliding_window", gw.U32, 1024),
             ("gemma4.attention.shared_kv_layers", gw.U32, 4), ("gemma4.attention.layer_norm_rms_epsilon", gw.F32, 1e-5),
             ("gemma4.final_logit_softcapping", gw.F32, 25.0), ("gemma4.embedding_length_per_layer_input", gw.U32, 256),
             ("gemma4.rope.freq_base", gw.F32, 5e5), ("gemma4.rope.freq_base_swa", gw.F32, 2e4),
             ("gemma4.feed_forward_length", gw.ARR, (gw.U32, [1024 * (1 + i % 2) for i in range(12)])),
             ("gemma4.attention.sliding_window_pattern", gw.ARR, (gw.BOOL, [i % 4 != 3 for i in range(12)]))]
    tensors = [("token_embd.weight", GgmlType.F16, (1536, 777), np.zeros(1536 * 777, np.float16)),
               ("per_layer_model_proj.weight", GgmlType.F16, (8,), np.zeros(8, np.float16))]
    with hip.Gguf(_cfg_file(tmp_path, extra, tensors)) as g:
        cfg, ffn, swa = g.gemma4_config(128)
    assert (cfg["n_kv"], cfg["hd_full"], cfg["hd_swa"], cfg["sliding_window"], cfg["shared_kv_layers"], cfg["ple_dim"]) == (2, 256, 128, 1024, 4, 256)
    assert cfg["eps"] == np.float32(1e-5) and cfg["softcap"] == 25.0 and cfg["rope_theta_full"] == 5e5 and cfg["rope_theta_swa"] == 2e4
    assert cfg["vocab"] == 777 and ffn == [1024 * (1 + i % 2) for i in range(12)] and swa == [i % 4 != 3 for i in range(12)]
    with hip.Gguf(_cfg_file(tmp_path, [("gemma4.feed_forward_length", gw.U32, 2048)])) as g:
        assert g.gemma4_config(64)[1] == [2048] * 12
    with hip.Gguf(_cfg_file(tmp_path, [("gemma4.feed_forward_length", gw.ARR, (gw.U32, [1, 2, 3]))])) as g:
        assert g.gemma4_config(64)[1] == [6144] * 12           # a list of the wrong length falls back


def test_config_from_gguf_errors(tmp_path):
    p = str(tmp_path / "e.gguf")
    t = [("x", GgmlType.F32, (8,), np.zeros(8, np.float32))]
    gw.write(p, [("general.architecture", gw.STR, "llama")], t)
    with hip.Gguf(p) as g, pytest.raises(hip.KshError, match="unsupported GGUF architecture `llama`"):
        g.gemma4_config(64)
    with hip.Gguf(_cfg_file(tmp_path, [("gemma4.expert_count", gw.U32, 8)])) as g, pytest.raises(hip.KshError, match="MoE"):
        g.gemma4_config(64)
    with hip.Gguf(_cfg_file(tmp_path, [("gemma4.attention.head_count_kv", gw.ARR, (gw.U32, [1, 2]))])) as g, \
            pytest.raises(hip.KshError, match="per-layer head_count_kv"):
        g.gemma4_config(64)
    with hip.Gguf(_cfg_file(tmp_path, [("gemma4.attention.head_count_kv", gw.U32, 3)])) as g, pytest.raises(hip.KshError, match="not divisible"):
        g.gemma4_config(64)
    gw.write(p, [("general.architecture", gw.STR, "gemma4")], t)
    with hip.Gguf(p) as g, pytest.raises(hip.KshError, match="block_count"):
        g.gemma4_config(64)


def test_reader_survives_every_truncation_and_header_mutation(tmp_path):
    """A damaged file is either refused with an error or opened with every tensor inside the mapping: each
    prefix of a small file, bytes of its header overwritten at random, and 8-byte fields blown up."""
    rng = np.random.default_rng(11)
    meta = [("x", gw.U32, 7), ("s", gw.STR, "hello"), ("arr", gw.ARR, (gw.U32, [1, 2, 3])), ("n", gw.ARR, (gw.STR, ["a", "bc"]))]
    tensors = [("t.f32", GgmlType.F32, (8, 4), rng.normal(size=32).astype(np.float32)),
               ("t.q4k", GgmlType.Q4_K, (256, 2), rng.integers(0, 256, 288, dtype=np.uint8)),
               ("t.q8_0", GgmlType.Q8_0, (32, 2), rng.integers(0, 256, 68, dtype=np.uint8))]
    base = tmp_path / "base.gguf"
    data_off = gw.write(str(base), meta, tensors)
    raw = base.read_bytes()
    variants = [raw[:cut] for cut in range(len(raw))]
    for _ in range(400):
        b = bytearray(raw)
        for _ in range(int(rng.integers(1, 4))):
            b[int(rng.integers(0, data_off))] = int(rng.integers(0, 256))
        variants.append(bytes(b))
    for _ in range(200):
        b = bytearray(raw)
        p = int(rng.integers(0, data_off - 8))
        b[p:p + 8] = [2**63, 2**64 - 1, 2**40, 2**32, 2**31][int(rng.integers(0, 5))].to_bytes(8, "little")
        variants.append(bytes(b))
    path = tmp_path / "v.gguf"
    opened = refused = 0
    for v in variants:
        path.write_bytes(v)
        try:
            g = hip.Gguf(str(path))
        except hip.KshError:
            refused += 1
            continue
        opened += 1
        for name in g.tensor_names():
            try:
                _, dims, view = g.tensor(name)
            except hip.KshError:                 # a name that is no longer valid UTF-8 cannot be asked for from here
                continue
            int(view.sum())                      # every byte the reader hands out is readable
        g.get_u32("x"), g.get_str("s"), g.get_list("arr"), g.get_list("n")
        g.close()
    assert refused >= len(raw) - 64 and opened >= 1     # prefixes short of the data section are all refused
