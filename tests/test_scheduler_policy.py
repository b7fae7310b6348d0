"""Host-side pool-pressure policy (morphserve_amd.server.scheduler) against scenarios worked
out by hand from MorphServe/server/scheduler.py: admission, growth by segments, give-back
thresholds, eviction order and swap-in.  No GPU: the pool actions are counters."""
import pytest

from helpers import Cfg
from morphserve_amd.server.scheduler import Request, RequestIdManager, Scheduler


class FakeEngine:
    """Counts pool actions; grows/shrinks the scheduler's budget as memory_utils does."""

    def __init__(self, num_gpu_blocks, seg, layers=8, quant_serve=True, per_step=2, floor=0, **cfg):
        self.engine_config = Cfg(block_size=16, max_batch_size=8, max_tokens_in_batch=4096, num_cpu_blocks=64,
                                 max_seqs_in_block_table=16, quant_serve=quant_serve,
                                 num_layers_to_quantize=per_step, num_layers_to_quantize_max=floor)
        self.engine_config.__dict__.update(cfg)
        bm = Cfg(num_free_blocks=num_gpu_blocks)
        self.model = Cfg(kv_cache_new_block_size=seg, next_unquantized_layer=layers - 1, layer_quant_list=[],
                         gpu_block_manager=bm)
        self.grows = self.give_backs = 0
        self.refuse_give_back = False
        self.scheduler = Scheduler(None, self.engine_config, num_gpu_blocks, grow=self.grow,
                                   give_back=self.give_back)

    def grow(self, engine):
        assert engine is self
        m = self.model
        m.layer_quant_list.append(m.next_unquantized_layer)
        m.next_unquantized_layer -= 1
        m.gpu_block_manager.num_free_blocks += m.kv_cache_new_block_size
        self.scheduler.num_gpu_blocks += m.kv_cache_new_block_size
        self.grows += 1

    def give_back(self, engine):
        if self.refuse_give_back:
            return False
        m = self.model
        m.next_unquantized_layer += 1
        m.layer_quant_list.remove(m.next_unquantized_layer)
        m.gpu_block_manager.num_free_blocks -= m.kv_cache_new_block_size
        self.scheduler.num_gpu_blocks -= m.kv_cache_new_block_size
        self.give_backs += 1
        return True


def test_request_ids_smallest_first_and_reuse():
    ids = RequestIdManager(3)
    assert [ids.get_id(), ids.get_id()] == [0, 1]
    ids.free_id(0)
    assert ids.get_id() == 0 and ids.get_id() == 2
    with pytest.raises(RuntimeError, match="No more available request ids"):
        ids.get_id()


def test_segments_short_is_a_ceiling_division_that_goes_negative():
    e = FakeEngine(10, 4)
    s = e.scheduler
    s.num_decoding_gpu_blocks = 8
    # 8 running + extra - 10 available, in segments of 4, rounded up
    assert [s.segments_short(x, 4) for x in (0, 2, 3, 6, 7, 11)] == [0, 0, 1, 1, 2, 3]
    s.num_decoding_gpu_blocks = 1
    assert s.segments_short(0, 4) == -2 and s.segments_short(4, 4) == -1     # floor division of the deficit


def test_plain_fcfs_admission_eviction_and_swap_in():
    e = FakeEngine(10, 4, quant_serve=False)
    s = e.scheduler
    r = [Request(prompt_len=64) for _ in range(3)]          # 4 blocks each
    s.on_requests_arrival(r)
    batch, sin, sout = s.get_next_batch(e)
    assert batch == r[:2] and not sin and not sout          # the third would need 12 > 10 blocks
    assert [x.request_id for x in r] == [0, 1, -1] and s.num_decoding_gpu_blocks == 8
    batch, sin, sout = s.get_next_batch(e)                  # head of line still blocked -> decode batch
    assert batch is s.running_q and batch == r[:2] and not sin and not sout
    for x in r[:2]:
        x.output_len = 17                                   # 81 tokens -> 6 blocks each: 12 > 10
    batch, sin, sout = s.get_next_batch(e)
    assert sout == [r[1]] and batch == [r[0]] and list(s.swapped_q) == [r[1]]   # newest evicted
    assert s.num_decoding_gpu_blocks == 6
    batch, sin, sout = s.get_next_batch(e)                  # evicted sequences block new prefills
    assert batch == [r[0]] and not sin and not sout and list(s.waiting_q) == [r[2]]
    r[0].max_output_len = 17
    s.on_batch_finish(batch)
    assert s.running_q == [] and s.request_id_manager.available_ids[-1] == 0
    batch, sin, sout = s.get_next_batch(e)
    assert sin == [r[1]] and batch == [r[1]] and not s.swapped_q and s.num_decoding_gpu_blocks == 6
    assert e.grows == 0 and e.give_backs == 0


def test_eviction_keeps_arrival_order_at_the_front_of_the_swapped_queue():
    e = FakeEngine(12, 4, quant_serve=False)
    s = e.scheduler
    r = [Request(prompt_len=48) for _ in range(4)]          # 3 blocks each = 12
    s.on_requests_arrival(r)
    s.get_next_batch(e)
    old = Request(prompt_len=16)
    s.swapped_q.append(old)                                 # somebody evicted earlier
    for x in r:
        x.output_len = 17                                   # 65 tokens -> 5 blocks each: 20 > 12
    batch, sin, sout = s.get_next_batch(e)
    assert sout == [r[2], r[3]] and batch == r[:2]
    assert list(s.swapped_q) == [r[3], r[2], old]           # extendleft of the arrival-ordered list


def test_prefill_admission_spends_the_whole_growth_budget_at_once():
    e = FakeEngine(10, 4, per_step=2, floor=1, layers=6)
    s = e.scheduler
    s.running_q = [Request(prompt_len=128, request_id=9)]
    s.num_decoding_gpu_blocks = 8
    a, b, c = Request(prompt_len=64), Request(prompt_len=160), Request(prompt_len=16)
    s.on_requests_arrival([a, b, c])
    batch, _, _ = s.get_next_batch(e)
    # a: 8 + 4 - 10 = 2 short -> 1 segment <= budget 2, layer 5 >= floor 1 and 5 - 1 >= 0:
    # BOTH budgeted segments are added (18 blocks).  b: 4 + 10 + 8 - 18 = 4 -> 1 segment but
    # the budget is spent -> stop; c stays behind b (head-of-line).
    assert batch == [a] and e.grows == 2 and s.num_gpu_blocks == 18
    assert list(s.waiting_q) == [b, c] and s.num_decoding_gpu_blocks == 12
    assert e.give_backs == 0                                # growth happened: no give-back in this call


def test_prefill_growth_refused_below_the_layer_floor_or_beyond_the_budget():
    e = FakeEngine(10, 4, per_step=2, floor=3, layers=3)    # next layer 2 < floor 3
    s = e.scheduler
    s.num_decoding_gpu_blocks = 8
    s.on_requests_arrival([Request(prompt_len=64)])
    batch, sin, sout = s.get_next_batch(e)
    assert batch == [] and e.grows == 0 and len(s.waiting_q) == 1
    e = FakeEngine(10, 4, per_step=2, floor=0, layers=8)
    s = e.scheduler
    s.num_decoding_gpu_blocks = 8
    s.on_requests_arrival([Request(prompt_len=16 * 11)])    # 11 + 8 - 10 = 9 -> 3 segments > budget 2
    batch, _, _ = s.get_next_batch(e)
    assert batch == [] and e.grows == 0
    e = FakeEngine(10, 4, per_step=4, floor=0, layers=2)    # 3 segments needed, layer 1 - 3 < 0
    s = e.scheduler
    s.num_decoding_gpu_blocks = 8
    s.on_requests_arrival([Request(prompt_len=16 * 11)])
    batch, _, _ = s.get_next_batch(e)
    assert batch == [] and e.grows == 0


def test_decode_pressure_grows_one_segment_at_a_time_then_evicts():
    e = FakeEngine(10, 4, per_step=2, layers=1)             # a single layer left to replace
    s = e.scheduler
    r = [Request(prompt_len=80, request_id=i) for i in range(2)]
    for x in r:
        x.output_len = 33                                   # 113 tokens -> 8 blocks each: 16 > 10
    s.running_q = list(r)
    batch, sin, sout = s.get_next_batch(e)
    # first pass: layer 0 available -> +4 (14 < 16); second pass: no layer left -> evict the newest
    assert e.grows == 1 and s.num_gpu_blocks == 14 and sout == [r[1]] and batch == [r[0]]
    assert e.give_backs == 0


def test_give_back_thresholds():
    def run(free, segments=3, waiting=False, refuse=False):
        e = FakeEngine(100, 4, per_step=2, layers=8)
        for _ in range(segments):
            e.grow(e)
        e.grows = 0
        e.model.gpu_block_manager.num_free_blocks = free
        e.refuse_give_back = refuse
        if waiting:
            e.scheduler.waiting_q.append(Request(prompt_len=16))
        e.scheduler.try_quant2org(e)
        return e.give_backs
    assert run(7) == 0            # needs >= 2 segments' worth (8) free to start
    assert run(8) == 1            # 8 > 4 -> give back (4 left); 4 > 4 fails
    assert run(9) == 2            # 9 -> 5 -> 1
    assert run(100) == 2          # never more than num_layers_to_quantize per call
    assert run(100, segments=1) == 1
    assert run(100, segments=0) == 0
    assert run(100, waiting=True) == 0
    assert run(100, refuse=True) == 0


def test_give_back_runs_only_in_calls_without_growth_or_swap_in():
    e = FakeEngine(16, 4, per_step=2, layers=8)
    s = e.scheduler
    e.grow(e)
    e.grow(e)                                               # 24 blocks, all free
    e.grows = 0
    s.running_q = [Request(prompt_len=16, request_id=0)]
    s.swapped_q.append(Request(prompt_len=16, request_id=1))
    batch, sin, sout = s.get_next_batch(e)
    assert len(sin) == 1 and e.give_backs == 0              # a swap-in suppresses the give-back
    batch, sin, sout = s.get_next_batch(e)
    assert not sin and e.give_backs == 2 and s.num_gpu_blocks == 16


@pytest.mark.parametrize("seed,quant_serve", [(0, True), (1, True), (2, False), (3, True), (4, False), (5, True)])
def test_random_serving_run_keeps_the_books(seed, quant_serve):
    """Random arrivals through the whole policy: every step the queues are disjoint, the running
    set fits the budget, ids are unique, segments grown and given back balance, arrival order is
    kept by admission, and every request finishes."""
    import random
    rnd = random.Random(seed)
    seg, layers = 6, 6
    e = FakeEngine(24, seg, layers=layers, quant_serve=quant_serve, per_step=2)
    s = e.scheduler
    all_reqs, admitted_order, pending = [], [], []
    for _ in range(60):
        pending.append(Request(prompt_len=rnd.choice([5, 16, 17, 40, 64, 100]), max_output_len=rnd.randint(1, 40)))
    steps = 0
    while (pending or s.waiting_q or s.running_q or s.swapped_q) and steps < 5000:
        steps += 1
        if pending and rnd.random() < 0.5:
            burst = [pending.pop() for _ in range(min(len(pending), rnd.randint(1, 4)))]
            all_reqs.extend(burst)
            s.on_requests_arrival(burst)
        # the block manager's free count as the engine would have left it: everything the
        # running sequences have stored so far is allocated (evicted ones sit in host memory)
        e.model.gpu_block_manager.num_free_blocks = s.num_gpu_blocks - sum(
            -(-(r.prompt_len + max(r.output_len - 1, 0)) // 16) for r in s.running_q)
        given_back_before = e.give_backs
        batch, sin, sout = s.get_next_batch(e)
        is_prefill = batch is not s.running_q
        if is_prefill:
            assert not sin and not sout
            admitted_order.extend(batch)
        for r in batch:                                   # one token per scheduled sequence
            r.output_len += 1
        # -- the books ------------------------------------------------------------------
        running, waiting, swapped = set(map(id, s.running_q)), set(map(id, s.waiting_q)), set(map(id, s.swapped_q))
        assert not (running & waiting) and not (running & swapped) and not (waiting & swapped)
        assert len(s.running_q) <= e.engine_config.max_batch_size
        ids = [r.request_id for r in s.running_q] + [r.request_id for r in s.swapped_q]
        assert len(ids) == len(set(ids)) and all(0 <= i < e.engine_config.max_seqs_in_block_table for i in ids)
        if not is_prefill:
            need = sum(-(-(r.prompt_len + r.output_len - 1) // 16) for r in s.running_q)    # before this step's token
            # the fit is checked before the give-backs of the same call, which look at the block
            # manager's free count from before this step's allocations (scheduler.py:75-89, :232-233):
            # the budget the running set was fitted to is the one before those give-backs
            assert need <= s.num_gpu_blocks + seg * (e.give_backs - given_back_before)
        assert s.num_gpu_blocks == 24 + seg * len(e.model.layer_quant_list)
        assert e.grows - e.give_backs == len(e.model.layer_quant_list) <= layers
        assert quant_serve or e.grows == 0
        s.on_batch_finish(batch)
    assert steps < 5000, "the run did not drain"
    assert all(r.is_finished() for r in all_reqs) and len(all_reqs) == 60
    assert [id(r) for r in admitted_order] == [id(r) for r in all_reqs]      # head-of-line order of arrival
    assert len(s.request_id_manager.available_ids) == e.engine_config.max_seqs_in_block_table
