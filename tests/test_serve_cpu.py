"""The slot scheduler's rounds (crates/ksearch_cli/src/scheduler.rs:78-349) on the CPU: ksearch_amd/csrc/serve.cpp and
kv_pool.cpp linked against a mock model (tests/host_mock) whose next token is a fixed function of (token, position)
and which logs every bind_slot / prefill_chunk / decode_token_sampled the scheduler issues."""
import ctypes as C

import pytest

from ksearch_amd.hip import FINISH_REASONS, SERVE_STOP_FN, ServeCfg, ServeEvent
from tests import host_mock

VOCAB = 1000
NO_EOS = (0xFFFFFFFF, 0xFFFFFFFE)


class Call(C.Structure):
    _fields_ = [("kind", C.c_int32), ("slot", C.c_int32), ("pos", C.c_int32), ("n", C.c_int32), ("token", C.c_uint32),
                ("seed", C.c_uint32), ("temperature", C.c_float), ("min_p", C.c_float)]


@pytest.fixture(scope="module")
def L():
    lib = C.CDLL(host_mock.build())
    vp = C.c_void_p
    lib.mock_model_create.restype = vp
    lib.mock_model_create.argtypes = [C.c_int, C.c_int, C.c_int, C.c_uint32, C.c_int]
    lib.mock_model_destroy.argtypes = [vp]
    lib.mock_model_calls.argtypes = [vp, C.POINTER(Call), C.c_int]
    lib.mock_model_clear_calls.argtypes = [vp]
    lib.ksh_last_error.restype = C.c_char_p
    lib.ksh_kvpool_create.argtypes = [vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(vp)]
    lib.ksh_kvpool_destroy.argtypes = [vp]
    lib.ksh_kvpool_seq_len.argtypes = [vp, C.c_int]
    lib.ksh_kvpool_active_batch.argtypes = [vp, C.POINTER(C.c_int), C.c_int]
    lib.ksh_serve_default_cfg.argtypes = [C.POINTER(ServeCfg)]
    lib.ksh_serve_create.argtypes = [vp, vp, C.POINTER(ServeCfg), C.POINTER(vp)]
    lib.ksh_serve_destroy.argtypes = [vp]
    lib.ksh_serve_submit.argtypes = [vp, C.POINTER(C.c_uint32), C.c_size_t, C.c_size_t, C.c_float, C.c_float, C.c_uint32,
                                     C.POINTER(C.c_uint64)]
    lib.ksh_serve_cancel.argtypes = [vp, C.c_uint64]
    lib.ksh_serve_tick.argtypes = [vp]
    lib.ksh_serve_poll.restype = C.c_size_t
    lib.ksh_serve_poll.argtypes = [vp, C.POINTER(ServeEvent), C.c_size_t]
    lib.ksh_serve_error_text.restype = C.c_char_p
    lib.ksh_serve_error_text.argtypes = [vp]
    lib.ksh_serve_pending.argtypes = [vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]
    return lib


class Rig:
    """A mock model, a pool and a scheduler over them."""

    def __init__(self, L, pool_slots=4, max_seq=64, mode=0, constant=5, fail_pos=-1, stop=None, **cfg):
        self.L = L
        self.model = L.mock_model_create(max_seq, VOCAB, mode, constant, fail_pos)
        self.pool = C.c_void_p()
        # (the context is only handed on to the buffer calls, which the mock answers from host memory)
        assert L.ksh_kvpool_create(C.c_void_p(1), pool_slots, max_seq, 1, 32, 1, C.byref(self.pool)) == 0
        c = ServeCfg()
        assert L.ksh_serve_default_cfg(C.byref(c)) == 0
        assert (c.slots, c.prefill_chunk, c.prefill_tokens_per_tick, tuple(c.eos), c.use_graph) == (4, 256, 2048, (1, 106), 1)
        assert c.batched_decode == 3
        c.eos[0], c.eos[1] = cfg.pop("eos", NO_EOS)
        cfg.setdefault("batched_decode", 0)      # the reference's serial rounds unless a test asks for batched ones
        for k, v in cfg.items():
            setattr(c, k, v)
        self._stop = SERVE_STOP_FN(lambda user, req, tok: int(bool(stop(req, tok)))) if stop else SERVE_STOP_FN()
        c.stop = self._stop
        self.h = C.c_void_p()
        rc = L.ksh_serve_create(self.model, self.pool, C.byref(c), C.byref(self.h))
        if rc:
            raise RuntimeError(L.ksh_last_error().decode())
        L.mock_model_clear_calls(self.model)     # (create binds slot 0 once, to find a pool that does not fit)

    def submit(self, prompt, max_tokens, temperature=0.0, min_p=0.0, seed=1):
        p = (C.c_uint32 * max(1, len(prompt)))(*prompt)
        rid = C.c_uint64()
        assert self.L.ksh_serve_submit(self.h, p, len(prompt), max_tokens, temperature, min_p, seed, C.byref(rid)) == 0
        return rid.value

    def tick(self):
        assert self.L.ksh_serve_tick(self.h) == 0
        out, buf = [], (ServeEvent * 16)()
        while True:
            n = self.L.ksh_serve_poll(self.h, buf, 16)
            for e in buf[:n]:
                if e.kind == 0:
                    out.append(("token", e.request, e.token))
                elif e.kind == 1:
                    out.append(("done", e.request, FINISH_REASONS[e.reason], e.prompt_tokens, e.completion_tokens))
                else:
                    out.append(("error", e.request, self.L.ksh_serve_error_text(self.h).decode()))
            if n < 16:
                return out

    def pending(self):
        w, a = C.c_int(), C.c_int()
        self.L.ksh_serve_pending(self.h, C.byref(w), C.byref(a))
        return w.value, a.value

    def run(self, limit=10000):
        out = []
        for _ in range(limit):
            out += self.tick()
            if self.pending() == (0, 0):
                return out
        raise AssertionError("still busy")

    def calls(self, clear=True):
        buf = (Call * 4096)()
        n = self.L.mock_model_calls(self.model, buf, 4096)
        out = [(("bind", "prefill", "decode", "round")[c.kind], c.slot, c.pos, c.n) for c in buf[:n]]
        full = list(buf[:n])
        if clear:
            self.L.mock_model_clear_calls(self.model)
        return out, full

    def occupied(self):
        return self.L.ksh_kvpool_active_batch(self.pool, None, 0)

    def close(self):
        self.L.ksh_serve_destroy(self.h)
        self.L.ksh_kvpool_destroy(self.pool)
        self.L.mock_model_destroy(self.model)


def expected(prompt, n, max_seq=64):
    """The mock's continuation: next = (31 * token + 7 * pos + 1) % VOCAB, the last prompt token fed at len - 1."""
    out, tok, pos = [], prompt[-1], len(prompt) - 1
    while len(out) < n and pos < max_seq:
        tok = (31 * tok + 7 * pos + 1) % VOCAB
        out.append(tok)
        pos += 1
    return out


def split(events):
    toks, done, errs = {}, {}, {}
    for e in events:
        if e[0] == "token":
            toks.setdefault(e[1], []).append(e[2])
        elif e[0] == "done":
            assert e[1] not in done
            done[e[1]] = e[2:]
        else:
            errs[e[1]] = e[2]
    return toks, done, errs


def test_prefill_budget_chunks_and_round_robin(L):
    """scheduler.rs:243-303 tick by tick: nothing decoding -> a request may eat the whole budget; something
    decoding -> prefill_chunk per request; the cursor resumes where the last tick stopped."""
    r = Rig(L, slots=3, prefill_chunk=4, prefill_tokens_per_tick=10)
    p = [list(range(10 * i + 1, 10 * i + 9)) for i in range(3)]      # three prompts of 8: 7 prefill tokens each
    ids = [r.submit(q, 3) for q in p]
    assert r.tick() == []
    assert r.calls()[0] == [("bind", 0, 0, 0), ("prefill", 0, 0, 7), ("bind", 1, 0, 0), ("prefill", 1, 0, 3)]   # 7 + 3 = the budget
    ev = r.tick()
    assert ev == [("token", ids[0], expected(p[0], 1)[0])]
    # decode first (slot 0), then from the cursor (request 2): chunks of 4 while something decodes
    assert r.calls()[0] == [("bind", 0, 7, 0), ("decode", 0, 7, 1), ("bind", 2, 0, 0), ("prefill", 2, 0, 4), ("bind", 1, 3, 0),
                            ("prefill", 1, 3, 4)]
    first = ev
    ev = r.tick()
    assert [e[1] for e in ev] == [ids[0], ids[1]]
    assert r.calls()[0] == [("bind", 0, 8, 0), ("decode", 0, 8, 1), ("bind", 1, 7, 0), ("decode", 1, 7, 1), ("bind", 2, 4, 0),
                            ("prefill", 2, 4, 3)]
    toks, done, errs = split(first + ev + r.run())
    assert not errs
    for i in range(3):
        assert toks[ids[i]] == expected(p[i], 3) and done[ids[i]] == ("length", 8, 3)
    assert r.occupied() == 0
    r.close()


def test_waiting_requests_are_admitted_as_slots_free_up(L):
    r = Rig(L, pool_slots=2, slots=2)
    p = [[3, 4, 5], [6, 7], [8], [9, 10, 11, 12]]
    n_new = [4, 2, 5, 3]
    ids = [r.submit(q, n) for q, n in zip(p, n_new)]
    seen_active = []
    events = []
    while r.pending() != (0, 0):
        events += r.tick()
        seen_active.append(r.pending())
        assert r.occupied() <= 2
    assert seen_active[0] == (2, 2)
    toks, done, _ = split(events)
    for i, rid in enumerate(ids):
        assert toks[rid] == expected(p[i], n_new[i]) and done[rid] == ("length", len(p[i]), n_new[i])
    # a one-token prompt has nothing to prefill: its only token is the first decode input
    calls, _ = r.calls()
    assert not any(c[0] == "prefill" and c[3] == 0 for c in calls)
    r.close()


def test_sampler_arguments_follow_the_request(L):
    """scheduler.rs:151, 184: the generator starts at seed | 1 and advances by 0x9E3779B9 before every token."""
    r = Rig(L)
    rid = r.submit([5, 6, 7], 4, temperature=0.7, min_p=0.1, seed=1234)
    toks, done, _ = split(r.run())
    _, full = r.calls()
    dec = [c for c in full if c.kind == 2]
    state = 1234 | 1
    for k, c in enumerate(dec):
        state = (state + 0x9E3779B9) & 0xFFFFFFFF
        assert c.seed == state and abs(c.temperature - 0.7) < 1e-7 and abs(c.min_p - 0.1) < 1e-7
        assert c.token == ([7] + toks[rid])[k] and c.pos == 2 + k
    assert len(dec) == 4 and done[rid] == ("length", 3, 4)
    r.close()


def test_stop_rules(L):
    prompt = [11, 12, 13, 14]
    full = expected(prompt, 12)
    assert len(set(full)) == 12
    # EOS: not emitted, reason "stop" (scheduler.rs:203-206)
    r = Rig(L, eos=(full[5], 0xFFFFFFFF))
    rid = r.submit(prompt, 12)
    toks, done, _ = split(r.run())
    assert toks[rid] == full[:5] and done[rid] == ("stop", 4, 5) and r.occupied() == 0
    r.close()
    # the host's stop callback, asked after the EOS check and before the token is counted
    asked = []
    r = Rig(L, eos=(full[7], 0xFFFFFFFF), stop=lambda req, tok: asked.append(tok) or tok == full[3])
    rid = r.submit(prompt, 12)
    toks, done, _ = split(r.run())
    assert toks[rid] == full[:3] and done[rid] == ("stop", 4, 3) and asked == full[:4]
    r.close()
    # max_tokens 0 counts as 1; max_seq ends a request with "length"
    r = Rig(L, max_seq=10)
    a, b = r.submit(prompt, 0), r.submit(prompt, 100)
    toks, done, _ = split(r.run())
    assert toks[a] == full[:1] and done[a] == ("length", 4, 1)
    assert toks[b] == expected(prompt, 100, max_seq=10) and len(toks[b]) == 7 and done[b] == ("length", 4, 7)
    r.close()
    # 24 equal tokens in a row: "stop", the 24th counted but not sent (scheduler.rs:219-222, 342-348)
    r = Rig(L, mode=1, constant=9)
    rid = r.submit(prompt, 50)
    toks, done, _ = split(r.run())
    assert toks[rid] == [9] * 23 and done[rid] == ("stop", 4, 24)
    r.close()


def test_errors_and_cancellation(L):
    prompt = [21, 22, 23]
    full = expected(prompt, 8)
    # a decode failure: error event with the text, no done event, slot freed, others unaffected
    r = Rig(L, mode=2, fail_pos=4, slots=1)
    a, b = r.submit(prompt, 8), r.submit([1, 2], 2)
    toks, done, errs = split(r.run())
    assert toks[a] == full[:2] and errs[a] == "mock decode failure at 4" and a not in done
    assert toks[b] == expected([1, 2], 2) and done[b] == ("length", 2, 2) and r.occupied() == 0
    r.close()
    # empty prompt, prompt beyond max_seq, pool smaller than `slots`
    r = Rig(L, pool_slots=1, slots=2, max_seq=16)
    e, long_, nofit = r.submit([], 3), r.submit([1] * 20, 3), r.submit(prompt, 2)
    toks, done, errs = split(r.run())
    assert errs[e] == "empty prompt" and errs[long_] == "max_seq exceeded" and long_ not in done
    # (asked for while the over-long request still held the only slot: scheduler.rs:150-158)
    assert errs[nofit] == "admit failed: KvPool full (max_batch=1)" and r.occupied() == 0
    ok = r.submit(prompt, 2)
    toks, done, errs = split(r.run())
    assert not errs and toks[ok] == full[:2] and done[ok] == ("length", 3, 2)
    r.close()
    # cancellation of a running and of a waiting request
    r = Rig(L, slots=1)
    a, b = r.submit(prompt, 8), r.submit(prompt, 8)
    ev = r.tick() + r.tick() + r.tick()
    assert L.ksh_serve_cancel(r.h, a) == 0 and L.ksh_serve_cancel(r.h, b) == 0
    ev += r.run()
    toks, done, _ = split(ev)
    assert toks[a] == full[:2] and done[a] == ("cancelled", 3, 3) and done[b] == ("cancelled", 3, 0) and b not in toks
    assert L.ksh_serve_cancel(r.h, a) == 1 and b"not queued or running" in L.ksh_last_error()
    r.close()
    # bad configuration
    with pytest.raises(RuntimeError, match="slots=0"):
        Rig(L, slots=0)


def test_destroy_frees_the_slots_of_running_requests(L):
    r = Rig(L, pool_slots=2, slots=2)
    r.submit([1, 2, 3], 30), r.submit([4, 5], 30)
    r.tick(), r.tick()
    assert r.occupied() == 2
    L.ksh_serve_destroy(r.h)
    assert r.occupied() == 0
    L.ksh_kvpool_destroy(r.pool)
    L.mock_model_destroy(r.model)


def test_batched_decode_rounds(L):
    """batched_decode = 2: two or more decoding requests take their step as one ksh_gemma4_decode_round (one record
    per row in the mock's log, n = rows of the round), a single one goes through bind_slot + decode_token_sampled as
    before; tokens, sampler seeds and stop rules are those of the serial rounds.  With the threshold at 3 the last two
    requests go one by one again."""
    prompts = [[5, 6, 7], [9, 10], [11, 12, 13, 14]]
    lens = [6, 3, 5]
    serial, batched = Rig(L, batched_decode=0), Rig(L, batched_decode=2)
    logs = {}
    for name, rig in (("serial", serial), ("batched", batched)):
        ids = [rig.submit(p, n, temperature=0.7 if i == 1 else 0.0, min_p=0.05, seed=40 + i) for i, (p, n) in enumerate(zip(prompts, lens))]
        toks, done, errs = split(rig.run())
        assert not errs
        for rid, p, n in zip(ids, prompts, lens):
            assert toks[rid] == expected(p, n) and done[rid][0] == "length"
        logs[name] = rig.calls()
        assert rig.occupied() == 0
    s_calls, s_full = logs["serial"]
    b_calls, b_full = logs["batched"]
    assert not any(c[0] == "round" for c in s_calls)
    rounds = [c for c in b_calls if c[0] == "round"]
    # 3 tokens by all three requests together, 2 more by the two longer ones, the last by the longest alone
    assert [c[3] for c in rounds] == [3] * 9 + [2] * 4
    assert sum(c[0] == "decode" for c in b_calls) == 1
    # every decoded token saw the same (slot, position, input token, seed, temperature, min_p) as in the serial rounds
    key = lambda c: (c.slot, c.pos, c.token, c.seed, round(c.temperature, 6), round(c.min_p, 6))
    assert sorted(key(c) for c in s_full if c.kind == 2) == sorted(key(c) for c in b_full if c.kind in (2, 3))
    serial.close()
    batched.close()
    three = Rig(L, batched_decode=3)
    ids = [three.submit(p, n) for p, n in zip(prompts, lens)]
    toks, done, errs = split(three.run())
    assert not errs and all(toks[r] == expected(p, n) for r, p, n in zip(ids, prompts, lens))
    calls, _ = three.calls()
    assert [c[3] for c in calls if c[0] == "round"] == [3] * 9 and sum(c[0] == "decode" for c in calls) == 2 * 2 + 1
    three.close()


def test_batched_decode_more_requests_than_a_round_holds_and_errors(L):
    """20 decoding requests are two rounds (16 + 4); a failing round sends an error to each of its requests and frees
    their slots."""
    rig = Rig(L, pool_slots=20, slots=20, batched_decode=2)
    ids = [rig.submit([3 + i, 4], 2) for i in range(20)]
    toks, done, errs = split(rig.run())
    assert not errs and all(toks[r] == expected([3 + i, 4], 2) for i, r in enumerate(ids))
    calls, _ = rig.calls()
    assert sorted({c[3] for c in calls if c[0] == "round"}) == [4, 16]
    rig.close()
    rig = Rig(L, mode=2, fail_pos=3, batched_decode=2)
    a, b = rig.submit([1, 2, 3], 5), rig.submit([4, 5, 6], 5)
    toks, done, errs = split(rig.run())
    assert set(errs) == {a, b} and all("mock decode failure" in errs[r] for r in (a, b))
    assert len(toks[a]) == 1 and len(toks[b]) == 1           # position 2 decoded, position 3 failed
    assert rig.occupied() == 0
    rig.close()
