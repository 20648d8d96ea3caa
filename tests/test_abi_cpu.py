"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, and its host-only parts (plan cache, schedule candidates,
descriptor plumbing, error reporting) behave like the reference's."""
import ctypes as C
import os
import re

import pytest

from ksearch_amd import hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "ksearch_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ksh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = C.CDLL(hip.LIB_PATH)
    names = header_symbols()
    assert len(names) >= 40
    for n in names:
        assert hasattr(L, n), f"{n} is declared in include/ksearch_hip.h but not exported"
    # and the Python binding covers the same set
    assert sorted(hip.SYMBOLS) == names


def _header_prototypes():
    """name -> number of parameters, from the header's declarations"""
    text = open(os.path.join(ROOT, "include", "ksearch_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for name, params in re.findall(r"(?m)^\s*(?:const\s+)?\w+(?:\s+const)?[\s\*]+(ksh_\w+)\s*\(([^;{)]*)\)\s*;", text):
        params = params.strip()
        out[name] = 0 if params in ("", "void") else params.count(",") + 1
    return out


def test_rust_listing_in_the_integration_notes_covers_the_header():
    """The binding a maintainer would add declares every function of the header with the
    header's number of parameters, and every structure the header defines by value."""
    protos = _header_prototypes()
    assert sorted(protos) == header_symbols()
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    rust = text[text.index("## 2. FFI declarations"):text.index("## 3.")]
    declared = {}
    for name, params in re.findall(r"pub fn (ksh_\w+)\(([^;]*?)\)\s*(?:->[^;]*)?;", rust, flags=re.S):
        params = params.strip()
        declared[name] = 0 if not params else len(re.findall(r"\b\w+\s*:", params))
    assert sorted(declared) == sorted(protos), sorted(set(protos) ^ set(declared))
    for name, n in protos.items():
        assert declared[name] == n, f"{name}: {declared[name]} parameters in the Rust listing, {n} in the header"
    header = open(os.path.join(ROOT, "include", "ksearch_hip.h")).read()
    for c_name in re.findall(r"\}\s*(ksh_\w+)\s*;", header):
        rust_name = "".join(w.capitalize() for w in c_name.split("_"))
        assert f"pub struct {rust_name} " in rust, f"{c_name} has no {rust_name} in the Rust listing"


def test_enums_match_header():
    text = open(os.path.join(ROOT, "include", "ksearch_hip.h")).read()
    for m in re.finditer(r"\b(KSH_[A-Z0-9_]+)\s*=\s*(\d+)", text):
        name, val = m.group(1)[4:], int(m.group(2))
        if name in hip.DType.__members__:
            assert hip.DType[name] == val
        elif name in hip.Kind.__members__:
            assert hip.Kind[name] == val
        elif name.startswith("GGML_"):
            assert hip.GgmlType[name[5:]] == val
        elif name == "LOAD_KEEP_Q6K":
            assert hip.LOAD_KEEP_Q6K == val
        elif name.startswith("SERVE_"):
            assert ("token", "done", "error")[val] == name[6:].lower()   # the kinds Serve.poll maps
        elif name.startswith("FINISH_"):
            assert hip.FINISH_REASONS[val] == name[7:].lower()
        else:
            raise AssertionError(f"KSH_{name} has no Python counterpart")


def test_struct_sizes():
    assert C.sizeof(hip.Sched) == 32
    assert C.sizeof(hip.KernelDesc) == 4 + 16 + 4 + 64 + 16 + 32     # kind, dtypes, pad, dims, params, sched
    assert C.sizeof(hip.GemmaCfg) == 48
    assert C.sizeof(hip.GemmaLayer) == 13 * 8
    assert C.sizeof(hip.Gemma4Cfg) == 11 * 4 + 6 * 4
    assert C.sizeof(hip.Gemma4Layer) == 11 * 4 + 4 + 16 * 8 + 8          # ints, pad, pointers, scale + tail pad
    assert C.sizeof(hip.Gemma4Globals) == 8 * 8
    assert C.sizeof(hip.ServeCfg) == 3 * 4 + 8 + 2 * 4 + 4 + 2 * 8          # ints, eos, use_graph + batched_decode, pad, pointers
    assert C.sizeof(hip.ServeEvent) == 8 + 5 * 4 + 4


def test_context_fails_loudly_without_gpu():
    if os.path.exists("/dev/kfd") and os.access("/dev/kfd", os.R_OK | os.W_OK):
        pytest.skip("a GPU is present")
    with pytest.raises(hip.KshError) as e:
        hip.Context()
    assert "HIP device" in str(e.value) or "gfx950" in str(e.value)


def test_plan_cache_roundtrip(tmp_path, monkeypatch):
    monkeypatch.setenv("KSEARCH_BEAM_CACHE", str(tmp_path / "beam"))
    dims = [4096, 4096]
    assert hip.plan_load("matvec_q4k", dims, "gfx950") is None
    s = hip.Sched(tg=256, vec=2, unroll=1, nsg=4, nr0=2, k_split=1, lds_tile=0)
    hip.plan_save("matvec_q4k", dims, "gfx950", s, 0.0123)
    key = hip.plan_key("matvec_q4k", dims, "gfx950")
    assert re.fullmatch(r"matvec_q4k_4096x4096_[0-9a-f]{16}", key)
    path = tmp_path / "beam" / f"{key}.txt"
    lines = dict(l.split("=") for l in path.read_text().split())
    # the reference's six keys, in its format (beam.rs:125-139), plus the two gfx950 ones
    assert lines["tg"] == "256" and lines["vec"] == "2" and lines["unroll"] == "1"
    assert lines["nsg"] == "4" and lines["nr0"] == "2" and lines["ms"] == "0.012300"
    got, ms = hip.plan_load("matvec_q4k", dims, "gfx950")
    assert got.as_dict() == s.as_dict() and abs(ms - 0.0123) < 1e-9
    # keyed by chip and dims
    assert hip.plan_load("matvec_q4k", dims, "other-chip") is None
    assert hip.plan_load("matvec_q4k", [4096, 2048], "gfx950") is None
    assert hip.plan_key("matvec_q4k", dims, "a") != hip.plan_key("matvec_q4k", dims, "b")


def test_plan_cache_reads_reference_format(tmp_path, monkeypatch):
    monkeypatch.setenv("KSEARCH_BEAM_CACHE", str(tmp_path))
    key = hip.plan_key("matvec_q6k", [262144, 2048], "gfx950")
    # a file as the reference writes it: no nsg/nr0 lines -> defaults 2 and 4 (beam.rs:112-121)
    (tmp_path / f"{key}.txt").write_text("tg=32\nvec=1\nunroll=2\nms=1.500000\n")
    s, ms = hip.plan_load("matvec_q6k", [262144, 2048], "gfx950")
    assert (s.tg, s.vec, s.unroll, s.nsg, s.nr0, ms) == (32, 1, 2, 2, 4, 1.5)
    # a file missing a mandatory key is no plan
    (tmp_path / f"{key}.txt").write_text("tg=32\nvec=1\n")
    assert hip.plan_load("matvec_q6k", [262144, 2048], "gfx950") is None


def test_plan_kinds_and_candidates():
    d = hip.make_desc(hip.Kind.MATVEC, (4096, 4096), (hip.DType.Q4K, hip.DType.F32))
    assert hip.plan_kind(d) == "matvec_q4k"
    assert hip.plan_kind(hip.make_desc(hip.Kind.MATVEC, (8, 2048), (hip.DType.Q6K,))) == "matvec_q6k"
    assert hip.plan_kind(hip.make_desc(hip.Kind.MATVEC_BATCH, (8, 2048, 16), (hip.DType.Q4K,))) == "mul_mm_q4k"
    assert hip.plan_kind(hip.make_desc(hip.Kind.MATVEC_BATCH, (8, 2048, 16), (hip.DType.Q6K,))) == "mul_mm_q6k"
    assert hip.plan_kind(hip.make_desc(hip.Kind.RMSNORM, (2048,))) is None
    c = hip.beam_candidates(d)
    assert len(c) >= 12
    assert len({tuple(s.as_dict().items()) for s in c}) == len(c)
    assert all(s.tg == 64 * s.nsg for s in c)
    assert hip.beam_candidates(hip.make_desc(hip.Kind.RMSNORM, (2048,))) == []
    # the prefill GEMM: whole rows, the small-batch form up to 64 tokens, K slices where the tiles are few
    mm = lambda batch, rows, cols, xdt: [(s.nr0, s.k_split) for s in hip.beam_candidates(
        hip.make_desc(hip.Kind.MATVEC_BATCH, (rows, cols, batch), (hip.DType.Q4K, xdt, hip.DType.F32)))]
    assert mm(512, 8192, 2048, hip.DType.BF16) == [(128, 1)]
    assert mm(256, 2048, 2048, hip.DType.F32) == [(128, 1), (128, 2), (128, 4)]
    assert mm(40, 2048, 1536, hip.DType.F32) == [(128, 1), (32, 8), (128, 2)]
