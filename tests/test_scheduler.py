"""The scheduler's decisions, with the cache manager's host bookkeeping and made-up tokens (CPU).
Cases follow the reference's tests/zedinfer/test_scheduler_sampling.cpp."""
import pytest
import torch

from zedinfer_amd.cache import CacheManager
from zedinfer_amd.config import SchedulerConfig
from zedinfer_amd.engine.request import GenerationConfig, InferenceRequest, RequestPhase, resolve_max_new_tokens
from zedinfer_amd.engine.scheduler import QueueFull, Scheduler
from zedinfer_amd.parts.mixers import attention_cache_request


def make(pages=64, page_size=4, **kw):
    cfg = SchedulerConfig(num_kv_blocks=pages, kv_block_size=page_size, **kw)
    cache = CacheManager({0: attention_cache_request("full", 1, 16)}, {}, pages, page_size, cfg.max_batch_requests,
                         torch.float32, None, cfg.max_batch_tokens)
    return Scheduler(cfg, cache, stop_token_ids=[99]), cache


def run_step(sched, cache, token=7):
    """What the serving loop does around a model step, with a constant 'sampled' token."""
    batch = sched.schedule()
    if batch.empty():
        return batch
    for e in batch.entries():
        cache.ensure(e.seq, e.seq.length + len(e.tokens))
        cache.commit(e.seq, e.seq.length + len(e.tokens))
    toks = token if isinstance(token, list) else [token] * len(batch.sampled_requests())
    sched.process_results(batch, toks)
    cache.check()
    return batch


def req(n, max_new=4, **kw):
    return InferenceRequest(list(range(1, n + 1)), GenerationConfig(max_new_tokens=max_new, **kw))


def test_mixed_batch_decode_rows_first_and_last_row_of_prompt():
    # reference: test_scheduler_sampling.cpp:64-102
    s, c = make()
    a = req(5)
    s.submit(a)
    b1 = run_step(s, c)
    assert b1.prefill_requests == [a] and b1.prefill_chunk_sizes == [5] and not b1.decode_requests
    assert a.phase == RequestPhase.DECODE and a.output_ids == [7] and a.generated_count == 1
    b = req(6)
    s.submit(b)
    batch = s.schedule()
    assert batch.decode_requests == [a] and batch.prefill_requests == [b]
    entries = batch.entries()
    assert entries[0].tokens == [7] and list(entries[0].want) == [0]           # the decode row comes first
    assert entries[1].tokens == [1, 2, 3, 4, 5, 6] and list(entries[1].want) == [5]   # last row of the prompt
    assert batch.sampled_requests() == [a, b]


def test_chunked_prefill_under_the_budget():
    s, c = make(max_batch_tokens=16, max_prefill_tokens=8)
    a, b = req(20, max_new=3), req(3, max_new=3)
    s.submit(a)
    s.submit(b)
    sizes = []
    for _ in range(3):
        batch = run_step(s, c)
        sizes.append((list(batch.prefill_chunk_starts), list(batch.prefill_chunk_sizes), len(batch.decode_requests)))
        assert batch.num_tokens() <= 16
    # a is cut 8 + 8 + 4; only when a's prompt completes does b get the rest of the budget (3 of 4 left)
    assert sizes == [([0], [8], 0), ([8], [8], 0), ([16, 0], [4, 3], 0)]
    assert a.output_ids == [7] and b.output_ids == [7]
    batch = run_step(s, c)
    assert len(batch.decode_requests) == 2 and not batch.prefill_requests
    # an unfinished prompt yields no token and stays at the head of the queue
    s2, c2 = make(max_prefill_tokens=4)
    x = req(10)
    s2.submit(x)
    b2 = s2.schedule()
    assert b2.sampled_requests() == [] and list(b2.entries()[0].want) == [] and s2.waiting[0] is x
    assert x.phase == RequestPhase.PREFILL


def test_decode_budget_and_request_cap():
    s, c = make(max_batch_requests=2)
    rs = [req(2, max_new=8) for _ in range(3)]
    for r in rs:
        s.submit(r)
    run_step(s, c)
    assert [r.phase for r in rs] == [RequestPhase.DECODE, RequestPhase.DECODE, RequestPhase.QUEUED]
    batch = run_step(s, c)
    assert len(batch.decode_requests) == 2 and not batch.prefill_requests       # the cap keeps the third out


def test_finish_reasons_and_release():
    s, c = make()
    a, b, d = req(3, max_new=2), req(3, max_new=5), req(3, max_new=1)
    for r in (a, b, d):
        s.submit(r)
    run_step(s, c, token=[7, 99, 7])
    assert b.done and b.finish_reason == "stop" and b.result.output_ids == [99]
    assert d.done and d.finish_reason == "length"                  # max_new_tokens == 1 ends at the prompt
    run_step(s, c)
    assert a.done and a.finish_reason == "length" and a.output_ids == [7, 7]
    assert not c.live and c.groups[0].pool.num_free == 64 and not s.has_work()
    e = req(3, max_new=3, ignore_eos=True)
    s.submit(e)
    for _ in range(3):
        run_step(s, c, token=99)
    assert e.finish_reason == "length" and e.output_ids == [99, 99, 99]


def test_request_that_can_never_fit_fails_instead_of_waiting():
    # reference: test_scheduler_sampling.cpp:104-131
    s, c = make(pages=4, page_size=4)
    big, small = req(40, max_new=4), req(4, max_new=2)
    s.submit(big)
    s.submit(small)
    batch = s.schedule()
    assert big.done and big.finish_reason == "error" and "Cannot admit" in big.error
    assert batch.prefill_requests == [small]                       # the queue moves on


def test_head_of_queue_waits_while_others_run():
    s, c = make(pages=8, page_size=4, generation_reserve=4)
    a = req(20, max_new=4)                                         # 24 tokens: 6 of 8 pages
    b = req(12, max_new=4)                                         # 16 tokens: 4 pages, does not fit beside a
    s.submit(a)
    run_step(s, c)
    s.submit(b)
    for _ in range(2):
        batch = run_step(s, c)
        assert batch.decode_requests == [a] and not batch.prefill_requests and b.phase == RequestPhase.QUEUED
    run_step(s, c)                                                 # a reaches its 4 tokens and frees its pages
    assert a.done
    batch = run_step(s, c)
    assert batch.prefill_requests == [b] and not b.error


def test_decode_exhaustion_fails_only_that_request():
    # reference: test_scheduler_sampling.cpp:133-170
    s, c = make(pages=4, page_size=4, generation_reserve=0)
    a, b = req(8, max_new=20), req(7, max_new=20)                  # promised 2 + 2 pages, all 4
    s.submit(a)
    s.submit(b)
    run_step(s, c)
    batch = run_step(s, c)                                         # a needs a third page: none unpromised
    assert a.done and a.finish_reason == "error" and "KV cache exhausted during decode" in a.error
    assert batch.decode_requests == [b]
    for _ in range(4):
        run_step(s, c)
    assert not b.done and b.generated_count == 6                   # b took over the pages a gave back
    c.check()


def test_queue_limit_and_limits_resolution():
    s, c = make(max_queue_size=2)
    s.submit(req(2))
    s.submit(req(2))
    with pytest.raises(QueueFull):
        s.submit(req(2))
    # reference: src/zedinfer/generation_types.cpp:39-61
    assert resolve_max_new_tokens(0, 100, 512) == 412
    assert resolve_max_new_tokens(1000, 100, 512) == 412
    assert resolve_max_new_tokens(5, 100, 512) == 5
    with pytest.raises(ValueError, match="no room"):
        resolve_max_new_tokens(5, 512, 512)
    s3, _ = make(max_seq_len=16)
    r = req(10, max_new=0)
    s3.submit(r)
    assert r.config.max_new_tokens == 6


def test_failed_step_fails_its_batch_and_frees():
    s, c = make()
    a = req(5)
    s.submit(a)
    batch = s.schedule()
    s.fail_batch(batch, "step failed: boom")
    assert a.done and a.error == "step failed: boom" and not c.live and not s.has_work()


def test_sampling_options_are_validated():
    # reference: tests/sampler/test_sampler.cpp:39-67
    s, _ = make()
    for bad in (dict(top_p=0.0), dict(top_p=1.5), dict(top_k=-1), dict(repetition_penalty=0.0),
                dict(temperature=-1.0)):
        with pytest.raises(ValueError):
            s.submit(req(2, **bad))
    with pytest.raises(ValueError, match="stream_callback"):
        s.submit(req(2, stream=True))


# ---- the batch after the one that runs ------------------------------------------------------

def commit(cache, batch):
    """What the engine does when it queues a step: the new tokens get their places."""
    for e in batch.entries():
        cache.ensure(e.seq, e.seq.length + len(e.tokens))
        cache.commit(e.seq, e.seq.length + len(e.tokens))


def test_batch_ahead_is_known_when_only_the_tokens_are_open():
    s, c = make()
    a, b = req(5, max_new=6), req(3, max_new=6)
    s.submit(a)
    s.submit(b)
    first = s.schedule()            # both prompts, whole
    commit(c, first)
    ahead = s.schedule_ahead(first)
    assert ahead is not None and ahead.decode_requests == [a, b] and ahead.tokens_on_device
    assert [list(e.want) for e in ahead.entries()] == [[0], [0]] and all(len(e.tokens) == 1 for e in ahead.entries())
    commit(c, ahead)
    s.process_results(first, [7, 8])
    assert a.output_ids == [7] and b.output_ids == [8]
    s.process_results(ahead, [9, 10])
    assert a.output_ids == [7, 9] and b.output_ids == [8, 10] and a.generated_count == 2
    # what the ordinary schedule makes next is the same kind of batch, with the tokens on the host
    nxt = s.schedule()
    assert nxt.decode_requests == [a, b] and [e.tokens for e in nxt.entries()] == [[9], [10]]
    c.check()


def test_no_batch_ahead_when_the_results_could_change_it():
    # the last token of a request: it ends with this step's result
    s, c = make()
    a = req(4, max_new=2)
    s.submit(a)
    first = s.schedule()
    commit(c, first)
    assert s.schedule_ahead(first) is not None          # 1 of 2 after this step
    s.process_results(first, [7])
    second = s.schedule()
    commit(c, second)
    assert s.schedule_ahead(second) is None             # 2 of 2 after this step
    # a cancelled request, and one whose sampling reads its history
    for kw, cancel in ((dict(), True), (dict(repetition_penalty=1.3, temperature=0.8), False)):
        s, c = make()
        a = req(4, max_new=8, **kw)
        s.submit(a)
        first = s.schedule()
        commit(c, first)
        a.cancelled = cancel
        assert s.schedule_ahead(first) is None
    # no page for the next token
    s, c = make(pages=2, page_size=4, generation_reserve=1)
    a = req(8, max_new=8)
    s.submit(a)
    first = s.schedule()
    commit(c, first)
    assert s.schedule_ahead(first) is None
    c.check()


def test_batch_ahead_takes_the_prompts_that_the_next_step_would():
    """The batch ahead holds, beside the decoding requests, the portions of prompts that ``schedule()`` would take
    after the running step: a prompt that is partly in goes on, a waiting prompt that fits is admitted, and a step
    that samples nothing (a portion in the middle of a prompt) has a batch ahead too."""
    # a prompt that is only partly in
    s, c = make(max_batch_tokens=8, max_prefill_tokens=8)
    a, b = req(3, max_new=8), req(12, max_new=8)
    s.submit(a)
    s.submit(b)
    first = s.schedule()            # a whole, 5 tokens of b
    assert first.prefill_chunk_sizes == [3, 5]
    commit(c, first)
    ahead = s.schedule_ahead(first)
    assert ahead.decode_requests == [a] and ahead.prefill_requests == [b] and ahead.tokens_on_device
    assert ahead.prefill_chunk_starts == [5] and ahead.prefill_chunk_sizes == [7] and ahead.sampled_requests() == [a, b]
    commit(c, ahead)
    s.process_results(first, [7])
    s.process_results(ahead, [8, 9])
    assert a.output_ids == [7, 8] and b.output_ids == [9] and b.phase == RequestPhase.DECODE
    c.check()
    # a waiting prompt that can be admitted now
    s, c = make()
    a, b = req(3, max_new=8), req(4, max_new=8)
    s.submit(a)
    first = s.schedule()
    commit(c, first)
    s.submit(b)
    ahead = s.schedule_ahead(first)
    assert ahead.decode_requests == [a] and ahead.prefill_requests == [b] and ahead.prefill_chunk_sizes == [4]
    # a portion in the middle of a prompt: nothing is sampled, the next portion is known all the same
    s, c = make(max_batch_tokens=8, max_prefill_tokens=8)
    a = req(20, max_new=8)
    s.submit(a)
    first = s.schedule()
    assert first.prefill_chunk_sizes == [8] and not first.sampled_requests()
    commit(c, first)
    ahead = s.schedule_ahead(first)
    assert ahead.prefill_chunk_starts == [8] and ahead.prefill_chunk_sizes == [8] and not ahead.decode_requests
    commit(c, ahead)
    s.process_results(first, [])
    s.process_results(ahead, [])
    last = s.schedule()
    assert last.prefill_chunk_starts == [16] and last.prefill_chunk_sizes == [4] and last.sampled_requests() == [a]
    c.check()


def test_requests_get_the_same_tokens_with_and_without_batches_ahead():
    """A random workload through the scheduler twice, once with every batch that can be made ahead made ahead (as
    the serving loop does), once without: prompts cut into portions, requests that end by length and on stop
    tokens, few pages.  The 'model' gives request r its k-th token as a function of (r, k) alone, so every
    request must get the same output either way; the cache's books must balance all along."""
    import random

    def run(ahead_on, seed):
        rng = random.Random(seed)
        s, c = make(pages=rng.choice([24, 40, 64]), page_size=4, max_batch_tokens=rng.choice([6, 12, 40]),
                    max_prefill_tokens=rng.choice([4, 8, 32]), max_batch_requests=rng.choice([2, 3, 8]),
                    generation_reserve=4)
        everyone = [req(rng.randint(1, 30), max_new=rng.randint(1, 12)) for _ in range(10)]
        late = everyone[7:]
        for r in everyone[:7]:
            s.submit(r)
        names = {id(r): i for i, r in enumerate(everyone)}

        def token(r):
            v = (names[id(r)] * 31 + len(r.output_ids) * 7) % 101
            return 99 if v % 17 == 0 else v            # now and then the stop token

        flight, steps, mixed_ahead = None, 0, 0
        while s.has_work() or flight is not None or late:
            steps += 1
            assert steps < 2000
            if late and (steps in (3, 9, 15) or not (s.has_work() or flight is not None)):
                s.submit(late.pop(0))
            if flight is None:
                batch = s.schedule()
                if batch.empty():
                    continue
                commit(c, batch)
            else:
                batch, flight = flight, None
            if ahead_on:
                nxt = s.schedule_ahead(batch)
                if nxt is not None:
                    commit(c, nxt)
                    flight = nxt
                    mixed_ahead += bool(nxt.prefill_requests)
            s.process_results(batch, [token(r) for r in batch.sampled_requests()])
            if flight is not None and not flight.prefill_requests and all(r.done for r in flight.decode_requests):
                flight = None
            c.check()
        assert not c.live and not late
        return [(r.finish_reason, r.error, list(r.result.output_ids) if r.result else None) for r in everyone], mixed_ahead

    mixed, reasons = 0, set()
    for seed in range(24):
        with_ahead, mixed_ahead = run(True, seed)
        without, _ = run(False, seed)
        assert with_ahead == without, seed
        mixed += mixed_ahead
        reasons |= {r[0] for r in without}
    assert mixed > 20                                   # batches ahead with portions of prompts were among them
    assert reasons >= {"stop", "length"}


def test_batch_ahead_while_the_head_of_the_queue_cannot_enter():
    s, c = make(max_batch_requests=1)
    a, b = req(3, max_new=8), req(3, max_new=8)
    s.submit(a)
    s.submit(b)
    first = s.schedule()
    assert first.prefill_requests == [a]
    commit(c, first)
    ahead = s.schedule_ahead(first)
    assert ahead is not None and ahead.decode_requests == [a]


def test_token_computed_for_a_request_that_ended_is_dropped():
    s, c = make()
    a, b = req(5, max_new=6), req(3, max_new=6)
    s.submit(a)
    s.submit(b)
    first = s.schedule()
    commit(c, first)
    ahead = s.schedule_ahead(first)
    commit(c, ahead)
    free_before = c.groups[0].pool.num_free
    s.process_results(first, [99, 8])                   # a ends on the stop token
    assert a.done and a.finish_reason == "stop" and a.result.output_ids == [99]
    assert c.groups[0].pool.num_free > free_before      # its pages are back while the step ahead still runs
    s.process_results(ahead, [5, 10])
    assert a.result.output_ids == [99] and b.output_ids == [8, 10]
    c.check()
    nxt = s.schedule()
    assert nxt.decode_requests == [b]


def test_token_computed_ahead_for_a_cancelled_request_is_dropped():
    s, c = make()
    a, b = req(5, max_new=6), req(3, max_new=6)
    s.submit(a)
    s.submit(b)
    first = s.schedule()
    commit(c, first)
    ahead = s.schedule_ahead(first)
    commit(c, ahead)
    s.process_results(first, [7, 8])
    a.cancelled = True                                  # for instance from its stream callback
    s.process_results(ahead, [9, 10])
    assert a.output_ids == [7] and b.output_ids == [8, 10]
    nxt = s.schedule()                                  # the ordinary schedule ends it
    assert a.done and a.finish_reason == "stop" and a.result.output_ids == [7] and nxt.decode_requests == [b]
    c.check()


# ---- what a request samples with when it sets nothing -----------------------------------------

def test_default_sampling_from_the_model_folder(tmp_path, monkeypatch):
    # reference: create_sampler_from_generation_config, src/zedinfer/engine.cpp:49-126
    import json
    from zedinfer_amd.sampling import default_sampling
    monkeypatch.delenv("ZEDINFER_FORCE_ARGMAX", raising=False)
    monkeypatch.delenv("ZEDINFER_REPETITION_PENALTY", raising=False)
    folder = str(tmp_path)
    assert default_sampling(folder).greedy                              # no file
    path = tmp_path / "generation_config.json"
    path.write_text(json.dumps(dict(do_sample=False, temperature=0.6)))
    assert default_sampling(folder).greedy
    path.write_text(json.dumps(dict(do_sample=True)))
    p = default_sampling(folder)
    assert (p.temperature, p.top_k, p.top_p, p.repetition_penalty, p.seed, p.greedy) == (1.0, 0, 1.0, 1.0, 0, False)
    path.write_text(json.dumps(dict(do_sample=True, temperature=0.6, top_k=20, top_p=0.95, repetition_penalty=1.05, seed=7)))
    p = default_sampling(folder)
    assert (p.temperature, p.top_k, p.top_p, p.repetition_penalty, p.seed) == (0.6, 20, 0.95, 1.05, 7)
    monkeypatch.setenv("ZEDINFER_REPETITION_PENALTY", "1.2")
    assert default_sampling(folder).repetition_penalty == 1.2
    monkeypatch.setenv("ZEDINFER_FORCE_ARGMAX", "1")
    assert default_sampling(folder).greedy
    monkeypatch.setenv("ZEDINFER_FORCE_ARGMAX", "0")
    assert not default_sampling(folder).greedy
    monkeypatch.delenv("ZEDINFER_REPETITION_PENALTY")
    path.write_text(json.dumps(dict(do_sample=True, top_p=1.5)))        # does not validate
    assert default_sampling(folder).greedy
    path.write_text("{ not json")
    assert default_sampling(folder).greedy


def test_requests_without_sampling_options_take_the_default():
    from zedinfer_amd.sampling import SamplingParams
    cfg = SchedulerConfig(num_kv_blocks=16, kv_block_size=4)
    cache = CacheManager({0: attention_cache_request("full", 1, 16)}, {}, 16, 4, cfg.max_batch_requests, torch.float32, None,
                         cfg.max_batch_tokens)
    s = Scheduler(cfg, cache, default_sampling=SamplingParams(temperature=0.6, top_k=20, seed=7))
    plain_req, own, greedy, seeded = req(3), req(3, temperature=0.9), req(3, use_argmax=True), req(3, seed=11)
    for r in (plain_req, own, greedy, seeded):
        s.submit(r)
    assert (plain_req.sampler.params.temperature, plain_req.sampler.params.top_k, plain_req.sampler.params.seed) == (0.6, 20, 7)
    assert (own.sampler.params.temperature, own.sampler.params.top_k) == (0.9, 0)
    assert greedy.sampler.params.greedy
    assert (seeded.sampler.params.temperature, seeded.sampler.params.seed) == (0.6, 11)
    # without a default: greedy, as before
    s2, _ = make()
    r = req(3)
    s2.submit(r)
    assert r.sampler.params.greedy


def test_bounds_that_many_decode_steps_share():
    """The bound of the sequences' lengths that sizes a decode step's attention launch (and keys its graph):
    never below the length, a power of two up to 1,024, then steps of 512 (of 2,048 beyond 8,192), so that a
    batch just past a power of two does not launch twice the workgroups it needs."""
    from zedinfer_amd.engine.engine import _bucket_at_least
    assert [_bucket_at_least(n, 256) for n in (1, 256, 257, 600, 1024)] == [256, 256, 512, 1024, 1024]
    assert [_bucket_at_least(n, 256) for n in (1025, 2049, 2560, 2561, 8192)] == [1536, 2560, 2560, 3072, 8192]
    assert [_bucket_at_least(n, 256) for n in (8193, 10240, 10241, 32768)] == [10240, 10240, 12288, 32768]
    last = 0
    for n in range(1, 40000, 37):
        b = _bucket_at_least(n, 256)
        assert b >= n and b >= last and (n <= 1024 or b - n < (512 if n <= 8192 else 2048))       # monotone, one step at most
        last = b


def test_sizes_at_which_a_serving_engine_measures_its_choices():
    """The multiples of the step that portions of prompts are padded to, from 128 rows to the most a step can
    bring, largest first; beyond 4,096 rows they lie further apart (32 an octave), and every number of rows has
    one at most a 32nd above it."""
    from zedinfer_amd.parts.rows import PORTION_ROWS, ProductRows, few_rows_entries, sizes_between
    from zedinfer_amd.parts.rows import many_rows as many_rows_size_at_least

    def many_rows_step_sizes(most):
        return sizes_between(ProductRows.step_rows, "mixed", 128, most)
    assert PORTION_ROWS == 64
    assert [ProductRows.step_rows(n, "portion") for n in (2, 64, 65, 200)] == [64, 64, 128, 256]
    assert many_rows_step_sizes(300) == [320, 256, 192, 128]
    assert many_rows_step_sizes(2112) == list(range(2112, 127, -64))
    assert many_rows_step_sizes(64) == [] and many_rows_step_sizes(100) == [128]
    assert many_rows_step_sizes(4300)[:4] == [4352, 4224, 4096, 4032]
    sizes = many_rows_step_sizes(20000)
    assert sizes[0] == 20480 and len(sizes) == 63 + 32 + 32 + 8
    for n in range(128, 20001, 7):
        up = many_rows_size_at_least(n)
        assert up in sizes and n <= up <= n + max(63, n // 32), n
    # what an engine measures by default: the sizes of its steps with prompt portions, and of its pure decode steps
    # of more than 64 requests
    from zedinfer_amd.engine import InferenceEngine
    decode_entries_at_least, rows = few_rows_entries, ProductRows.step_rows      # what a model of such parts answers
    few = InferenceEngine.default_warm_up_sizes(SchedulerConfig(max_batch_requests=8, max_batch_tokens=520, max_prefill_tokens=512), rows)
    # 520 tokens, rounded up, and one more size; then the decode steps of up to 8 requests
    assert few == [640, 576, 512, 448, 384, 320, 256, 192, 128, 64, 8, 4, 2, 1]
    many = InferenceEngine.default_warm_up_sizes(SchedulerConfig(max_batch_requests=200, max_batch_tokens=2248, max_prefill_tokens=2048), rows)
    assert many[0] == 2368 and [m for m in many if 64 < m <= 128] == [128, 112, 96, 80] and 224 in many and 160 in many
    assert len(many) == len(set(many)) and many[-8:] == [64, 48, 32, 16, 8, 4, 2, 1]
    for e in range(1, 201):
        assert decode_entries_at_least(e) in many
    long = InferenceEngine.default_warm_up_sizes(SchedulerConfig(max_batch_requests=8, max_batch_tokens=16392, max_prefill_tokens=16384,
                                                                 max_seq_len=32768), rows)
    assert long[:4] == [16896, 16384, 8448, 8192] and long[-5:] == [64, 8, 4, 2, 1]

    # a part that wants other numbers has its say: the model takes the least number that every part accepts
    from types import SimpleNamespace
    from zedinfer_amd.models.model import DecoderModel
    from zedinfer_amd.parts import Part

    class Tens(Part):
        def __init__(self):
            pass

        def step_rows(self, n, kind):
            return -(-n // 10) * 10

    class Products(Part):
        def __init__(self):
            pass
        step_rows = staticmethod(ProductRows.step_rows)
    model = SimpleNamespace(_row_parts=[Tens(), Products()], _step_rows={})
    assert DecoderModel.step_rows(model, 3, "decode") == 80          # the first multiple of 10 among 4, 8, 16, 32, 48, 64, 80
    assert DecoderModel.step_rows(model, 65, "portion") == 320       # ... and among the multiples of 64
    assert DecoderModel.step_rows(SimpleNamespace(_row_parts=[], _step_rows={}), 7, "decode") == 7


def test_a_recorded_shape_refuses_a_step_that_plans_differently():
    """A shape that has been recorded (tape or graph) keeps the launch sizes and the sizes of the index arrays that
    the mixers' planners gave its first step; a later step of the shape whose plan differs (a planner whose
    ``shape`` does not name all that its plan depends on) raises instead of running the wrong launches."""
    import numpy as np
    from types import SimpleNamespace
    from zedinfer_amd.engine.engine import Engine, _DecodeGraph
    from zedinfer_amd.parts.base import StepPlan

    def batch(tiles, n):
        return SimpleNamespace(plans={("attention", 16): StepPlan(arrays={"tile_entry": np.zeros(n, np.int32)},
                                                                  sizes={"num_tiles": tiles, "tile": 64})})
    dg = _DecodeGraph()
    Engine._same_plans(dg, batch(3, 3))
    Engine._same_plans(dg, batch(3, 3))
    with pytest.raises(RuntimeError, match="plans its launches differently"):
        Engine._same_plans(dg, batch(4, 3))
    with pytest.raises(RuntimeError, match="plans its launches differently"):
        Engine._same_plans(dg, batch(3, 5))
