"""The decode-before-prefill slot scheduler (crates/ksearch_cli/src/scheduler.rs:78-349) through the C ABI: each
request produces the tokens the model produces for it alone, admission / chunking / stop rules follow the
reference's rounds."""
import numpy as np
import pytest

import oracle
from ksearch_amd import hip, synth
from tests.test_gpu_gemma4 import FFN, PATTERN

pytestmark = pytest.mark.gpu

NO_EOS = (0xFFFFFFFF, 0xFFFFFFFE)   # ids no model emits: runs end by length


@pytest.fixture(scope="module")
def ctx():
    c = hip.Context()
    yield c
    c.close()


@pytest.fixture(scope="module")
def model(ctx):
    cfg = dict(synth.GEMMA4_TINY)
    w = synth.gemma4_weights(cfg, 610, oracle.quantize_q4k, oracle.quantize_q6k, ffn=FFN, swa_pattern=PATTERN, std=0.05)
    m = hip.Gemma4(ctx, cfg, w)
    yield m, cfg
    m.close()


def make_pool(ctx, cfg, slots):
    owners = cfg["n_layers"] - cfg["shared_kv_layers"]
    return hip.KvPool(ctx, slots, cfg["max_seq"], owners, max(cfg["hd_swa"], cfg["hd_full"]), cfg["n_kv"])


def alone(m, prompt, n_new):
    m.bind_slot(None, 0)
    m.reset()
    return m.generate(prompt, n_new, use_graph=True)[0]


def prompts_of(cfg, lens, seed):
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, cfg["vocab"], n)] for n in lens]


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


@pytest.mark.parametrize("use_graph,batched", [(True, 0), (False, 0), (True, 2)])
def test_three_requests_through_two_slots_equal_the_runs_alone(ctx, model, use_graph, batched):
    """batched = 2: whenever both slots decode, their step is one ksh_gemma4_decode_round (one pass over the weights
    for both); the tokens are still those of the runs alone."""
    m, cfg = model
    prompts = prompts_of(cfg, (5, 9, 3), 700)
    max_new = (10, 6, 8)
    want = [alone(m, p, n) for p, n in zip(prompts, max_new)]
    pool = make_pool(ctx, cfg, 2)
    sv = hip.Serve(m, pool, slots=2, prefill_chunk=4, prefill_tokens_per_tick=8, eos=NO_EOS, use_graph=use_graph, batched_decode=batched)
    ids = [sv.submit(p, n) for p, n in zip(prompts, max_new)]
    events = sv.tick()
    assert sv.pending() == (1, 2) and len(pool.active_batch()) == 2     # the third waits for a slot
    events += sv.run()
    toks, done, errs = split(events)
    assert not errs
    for i, rid in enumerate(ids):
        assert toks[rid] == want[i], i
        assert done[rid] == ("length", len(prompts[i]), max_new[i])
    assert pool.active_batch() == [] and sv.pending() == (0, 0)
    # the slots are clean for the next round of requests: same answers again
    ids2 = [sv.submit(p, n) for p, n in zip(prompts[::-1], max_new[::-1])]
    toks2, _, _ = split(sv.run())
    assert [toks2[r] for r in ids2] == want[::-1]
    sv.close()
    m.bind_slot(None, 0)
    pool.close()


def test_prefill_takes_small_chunks_while_something_decodes(ctx, model):
    """scheduler.rs:243-292: with nothing decoding a prefilling request eats the tick's budget, with a decoding
    request beside it only prefill_chunk tokens per tick; the prompt's last token is the first decode input."""
    m, cfg = model
    pa, pb = prompts_of(cfg, (2, 21), 701)
    pool = make_pool(ctx, cfg, 2)
    sv = hip.Serve(m, pool, slots=2, prefill_chunk=4, prefill_tokens_per_tick=8, eos=NO_EOS)
    ra, rb = sv.submit(pa, 12), sv.submit(pb, 3)
    seen_b, first_b_token_tick = [], None
    events = []
    for tick in range(1, 9):
        ev = sv.tick()
        events += ev
        seen_b.append(pool.seq_len(1))
        if first_b_token_tick is None and any(e[0] == "token" and e[1] == rb for e in ev):
            first_b_token_tick = tick
    # tick 1: A's one prefill token (budget 8 -> 7), B takes the 7 left; then 4 a tick while A decodes; 20 = the
    # prompt minus its last token; the decode tokens follow
    assert seen_b[:6] == [7, 11, 15, 19, 20, 21]
    assert first_b_token_tick == 6
    events += sv.run()
    toks, done, _ = split(events)
    assert toks[ra] == alone(m, pa, 12) and toks[rb] == alone(m, pb, 3)
    assert done[ra] == ("length", 2, 12) and done[rb] == ("length", 21, 3)
    sv.close()
    m.bind_slot(None, 0)
    pool.close()


def test_stop_rules_errors_and_cancellation(ctx, model):
    m, cfg = model
    # a prompt whose continuation has, at some position cut >= 2, a token that has not appeared before it (the tiny
    # random model repeats itself soon)
    for seed in range(702, 742):
        (p,) = prompts_of(cfg, (6,), seed)
        full = alone(m, p, 12)
        cut = next((i for i in range(2, 12) if full[i] not in full[:i]), None)
        if cut is not None:
            break
    assert cut is not None
    pool = make_pool(ctx, cfg, 2)

    # an EOS id ends the request with "stop" and is not emitted (scheduler.rs:203-206)
    sv = hip.Serve(m, pool, slots=2, eos=(full[cut], 0xFFFFFFFF))
    r = sv.submit(p, 12)
    toks, done, _ = split(sv.run())
    assert toks[r] == full[:cut] and done[r] == ("stop", 6, cut)
    sv.close()

    # the host's stop callback takes the place of the stop strings, at the same point of the round
    asked = []
    sv = hip.Serve(m, pool, slots=2, eos=NO_EOS, stop=lambda req, tok: asked.append((req, tok)) or tok == full[cut])
    r = sv.submit(p, 12)
    toks, done, _ = split(sv.run())
    assert toks[r] == full[:cut] and done[r] == ("stop", 6, cut)
    assert asked == [(r, t) for t in full[:cut + 1]]
    sv.close()
    sv = hip.Serve(m, pool, slots=2, eos=NO_EOS)

    # errors: an empty prompt at admission, a prompt beyond max_seq at its prefill; max_tokens 0 counts as 1
    r_empty, r_long, r_one = sv.submit([], 4), sv.submit([1] * (cfg["max_seq"] + 2), 4), sv.submit(p, 0)
    toks, done, errs = split(sv.run())
    assert errs[r_empty] == "empty prompt" and "max_seq exceeded" in errs[r_long]
    assert r_long not in done and toks[r_one] == full[:1] and done[r_one] == ("length", 6, 1)
    assert pool.active_batch() == []

    # a request that runs into max_seq ends with "length" (scheduler.rs:177-180)
    r = sv.submit(p, 1000)
    toks, done, _ = split(sv.run())
    if done[r][0] == "length":
        assert done[r] == ("length", 6, cfg["max_seq"] - 5) and len(toks[r]) == cfg["max_seq"] - 5
    else:
        # or it fell into a loop first: 24 equal tokens in a row end it, the 24th counted but not sent (scheduler.rs:219-222)
        assert done[r] == ("stop", 6, len(toks[r]) + 1) and len(set(toks[r][-23:])) == 1

    # cancellation: a running request finishes "cancelled" at its next token, a waiting one at once
    r1, r2, r3 = sv.submit(p, 12), sv.submit(p, 12), sv.submit(p, 12)
    ev = sv.tick() + sv.tick() + sv.tick()
    sv.cancel(r1)
    sv.cancel(r3)
    ev += sv.run()
    toks, done, _ = split(ev)
    assert done[r1][0] == "cancelled" and toks[r1] == full[:len(toks[r1])] and len(toks[r1]) < 12
    assert done[r3] == ("cancelled", 6, 0) and r3 not in toks
    assert toks[r2] == full and done[r2] == ("length", 6, 12)
    with pytest.raises(hip.KshError, match="not queued or running"):
        sv.cancel(r2)
    sv.close()
    m.bind_slot(None, 0)
    pool.close()


def test_sampled_requests_follow_the_host_sampler(ctx, model):
    """decode_token_sampled with temperature > 0: logits read back, sample_softcap_min_p with the request's
    generator state (seed | 1, advanced by 0x9E3779B9 before every token: scheduler.rs:151, 184)."""
    m, cfg = model
    (p,) = prompts_of(cfg, (7,), 703)
    temperature, min_p, seed, n_new = 0.9, 0.02, 1234, 10
    m.bind_slot(None, 0)
    m.reset()
    m.prefill_chunk(p[:-1])
    want, last, rng = [], p[-1], seed | 1
    for _ in range(n_new):
        rng = (rng + 0x9E3779B9) & 0xFFFFFFFF
        m.forward_token(last, want_logits=True, read_next=False)
        last = hip.sample_softcap_min_p(m.logits(), cfg["softcap"], temperature, min_p, rng)
        want.append(last)
    assert want != alone(m, p, n_new)        # the draw is not the argmax everywhere
    pool = make_pool(ctx, cfg, 1)
    sv = hip.Serve(m, pool, slots=1, eos=NO_EOS)
    r = sv.submit(p, n_new, temperature=temperature, min_p=min_p, seed=seed)
    toks, done, _ = split(sv.run())
    assert toks[r] == want and done[r] == ("length", 7, n_new)
    # the model's own entry point draws the same token
    m.bind_slot(None, 0)
    m.reset()
    m.prefill_chunk(p[:-1], use_graph=True)
    assert m.decode_token_sampled(p[-1], temperature, min_p, (seed | 1) + 0x9E3779B9) == want[0]
    sv.close()
    m.bind_slot(None, 0)
    pool.close()


def test_serve_create_errors(ctx, model):
    m, cfg = model
    owners = cfg["n_layers"] - cfg["shared_kv_layers"]
    bad = hip.KvPool(ctx, 1, cfg["max_seq"], owners + 1, 256, cfg["n_kv"])
    with pytest.raises(hip.KshError, match="kv layer mismatch"):
        hip.Serve(m, bad)
    bad.close()
    pool = make_pool(ctx, cfg, 1)
    with pytest.raises(hip.KshError, match="slots=0"):
        hip.Serve(m, pool, slots=0)
    # more slots asked for than the pool has: the request that finds no slot is told so (scheduler.rs:150-158)
    sv = hip.Serve(m, pool, slots=2, eos=NO_EOS)
    (p,) = prompts_of(cfg, (4,), 704)
    r1, r2 = sv.submit(p, 3), sv.submit(p, 3)
    toks, done, errs = split(sv.run())
    assert "admit failed: KvPool full" in errs[r2] and done[r1] == ("length", 4, 3)
    sv.close()
    m.bind_slot(None, 0)
    pool.close()


def test_a_token_repeated_24_times_ends_the_request(ctx):
    """scheduler.rs:219-222, 342-348: all-zero weights give all-zero logits, whose argmax is id 0 every time; the
    24th equal token in a row ends the request with "stop", counted in completion_tokens but not sent."""
    cfg = dict(synth.GEMMA4_TINY)
    w = synth.gemma4_weights(cfg, 611, oracle.quantize_q4k, oracle.quantize_q6k, ffn=FFN, swa_pattern=PATTERN, std=0.0)
    m = hip.Gemma4(ctx, cfg, w)
    pool = make_pool(ctx, cfg, 1)
    sv = hip.Serve(m, pool, slots=1, eos=NO_EOS)
    r = sv.submit([5, 6, 7], 40)
    toks, done, errs = split(sv.run())
    assert not errs and toks[r] == [0] * 23 and done[r] == ("stop", 3, 24)
    sv.close()
    pool.close()
    m.close()


def test_destroying_a_busy_scheduler_frees_its_slots(ctx, model):
    m, cfg = model
    pool = make_pool(ctx, cfg, 2)
    sv = hip.Serve(m, pool, slots=2, eos=NO_EOS)
    (p,) = prompts_of(cfg, (5,), 705)
    sv.submit(p, 30), sv.submit(p, 30), sv.submit(p, 30)
    sv.tick(), sv.tick()
    assert len(pool.active_batch()) == 2 and sv.pending() == (1, 2)
    sv.close()
    assert pool.active_batch() == []
    m.bind_slot(None, 0)
    pool.close()
