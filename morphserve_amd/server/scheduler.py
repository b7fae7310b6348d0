"""FCFS scheduler with the pool-pressure policy of MorphServe/server/scheduler.py.

Only the decisions that touch the KV pool are of interest here -- when a
prefill batch is admitted, when the pool must grow by a segment, when it may
give one back, and which sequences are evicted or brought back -- but they are
interleaved with the queueing, so the whole ``get_next_batch`` contract is kept
(same queues, same return triple, same counters).

The two pool actions are injected: ``grow(engine)`` stands where the reference
calls ``org2quant_and_update_kvcache`` (a weight layer is replaced by its
quantized twin and the freed bytes become one more KV segment) and
``give_back(engine) -> bool`` where it calls ``quant2org_and_update_kvcache``.
The defaults are this package's KV-only versions in ``memory_utils``; with
their ``migrate`` option a give-back no longer waits for the tail segment to
drain (the reference returns False then, memory_utils.py:623-624).
"""
from __future__ import annotations

import dataclasses
import time
from collections import deque
from typing import Callable, Deque, List, Optional, Tuple


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


@dataclasses.dataclass
class RequestMetrics:
    arrival_time: float = 0.0
    queued_time: float = 0.0


@dataclasses.dataclass
class Request:
    """The fields of MorphServe/server/structs.py::Request the scheduler reads."""
    prompt_len: int
    max_output_len: int = 1 << 30
    output_len: int = 0
    request_id: int = -1
    req_metrics: RequestMetrics = dataclasses.field(default_factory=RequestMetrics)

    def get_cur_output_len(self) -> int:
        return self.output_len

    def is_finished(self) -> bool:
        return self.output_len >= self.max_output_len


class RequestIdManager:
    """Ids in [0, max_id); the smallest unused id of a fresh manager goes out first and a
    returned id is the next one handed out (MorphServe/server/scheduler.py:11-36)."""

    def __init__(self, max_id: int):
        self.max_id = max_id
        self.available_ids = list(range(max_id - 1, -1, -1))

    def get_id(self) -> int:
        if not self.available_ids:
            raise RuntimeError("No more available request ids. Please try to increase `max_seqs_in_block_table`")
        return self.available_ids.pop()

    def free_id(self, req_id: int) -> None:
        self.available_ids.append(req_id)

    def free_ids(self, req_ids: List[int]) -> None:
        self.available_ids.extend(req_ids)


class Scheduler:
    """``get_next_batch(engine)`` -> (batch, newly_swapped_in, newly_swapped_out).

    ``engine`` is read exactly as the reference reads it:
    ``engine.engine_config.{quant_serve, num_layers_to_quantize, num_layers_to_quantize_max}``,
    ``engine.model.{kv_cache_new_block_size, next_unquantized_layer, layer_quant_list,
    gpu_block_manager.num_free_blocks}``.
    """

    def __init__(self, model_config, engine_config, num_gpu_blocks: int,
                 grow: Optional[Callable] = None, give_back: Optional[Callable] = None):
        self.model_config = model_config
        self.engine_config = engine_config
        self.num_gpu_blocks = num_gpu_blocks
        self.waiting_q: Deque[Request] = deque()
        self.running_q: List[Request] = []
        self.swapped_q: Deque[Request] = deque()          # evicted sequences, oldest first
        self.num_decoding_gpu_blocks = 0                  # blocks the running sequences need
        self.num_free_cpu_blocks = engine_config.num_cpu_blocks
        self.request_id_manager = RequestIdManager(engine_config.max_seqs_in_block_table)
        if grow is None or give_back is None:
            from . import memory_utils
            grow = grow or memory_utils.org2quant_and_update_kvcache
            give_back = give_back or memory_utils.quant2org_and_update_kvcache
        self._grow = grow
        self._give_back = give_back

    # -- small pieces -----------------------------------------------------------------
    def _get_block_needed(self, request: Request) -> int:
        return _cdiv(request.prompt_len + request.get_cur_output_len(), self.engine_config.block_size)

    def on_requests_arrival(self, requests: List[Request]) -> None:
        self.waiting_q.extend(requests)

    def segments_short(self, extra_blocks: int, seg_blocks: int) -> int:
        """How many more segments the pool needs before ``extra_blocks`` more blocks fit next
        to the running sequences; <= 0 when they fit (scheduler.py:114)."""
        deficit = extra_blocks + self.num_decoding_gpu_blocks - self.num_gpu_blocks
        return (deficit + seg_blocks - 1) // seg_blocks

    # -- giving segments back ---------------------------------------------------------
    def try_quant2org(self, engine) -> None:
        """Give segments back while the pool is comfortably empty (scheduler.py:75-89):
        only with nothing waiting and at least ``num_layers_to_quantize`` segments' worth of
        free blocks; then up to ``num_layers_to_quantize`` give-backs, each needing more
        than ``num_layers_to_quantize // 2`` segments' worth still free, stopping at the
        first refusal."""
        cfg, model = engine.engine_config, engine.model
        seg, per_step = model.kv_cache_new_block_size, cfg.num_layers_to_quantize
        if not model.layer_quant_list or self.waiting_q:
            return
        if not model.gpu_block_manager.num_free_blocks >= seg * per_step:
            return
        for _ in range(per_step):
            if model.layer_quant_list and model.gpu_block_manager.num_free_blocks > seg * (per_step // 2):
                if not self._give_back(engine):
                    break

    # -- the step ---------------------------------------------------------------------
    def get_next_batch(self, engine) -> Tuple[List[Request], List[Request], List[Request]]:
        cfg = engine.engine_config
        grow_budget = cfg.num_layers_to_quantize              # segments this call may still add
        if not self.swapped_q:
            batch, batch_blocks, grow_budget = self._admit_prefill(engine, grow_budget)
            if batch:
                now = time.perf_counter()
                for req in batch:
                    req.request_id = self.request_id_manager.get_id()
                    req.req_metrics.queued_time = now
                self.running_q.extend(batch)
                self.num_decoding_gpu_blocks += batch_blocks
                if cfg.quant_serve and grow_budget == cfg.num_layers_to_quantize:
                    self.try_quant2org(engine)
                return batch, [], []

        # decoding batch: first make the running set fit, then refill it from the evicted
        self.num_decoding_gpu_blocks = sum(self._get_block_needed(r) for r in self.running_q)
        evicted: List[Request] = []
        while len(self.running_q) > self.engine_config.max_batch_size or \
                self.num_decoding_gpu_blocks > self.num_gpu_blocks:
            if len(self.running_q) > self.engine_config.max_batch_size:
                raise RuntimeError("running set exceeds max_batch_size")   # the reference exits here
            if cfg.quant_serve and engine.model.next_unquantized_layer >= 0 and grow_budget > 0:
                self._grow(engine)                                        # scheduler.py:196-200
                grow_budget -= 1
            else:
                victim = self.running_q.pop()                             # newest first
                self.num_decoding_gpu_blocks -= self._get_block_needed(victim)
                evicted.append(victim)
        evicted.reverse()                                                 # back to arrival order

        returned: List[Request] = []
        if evicted:
            self.swapped_q.extendleft(evicted)
        else:
            while self.swapped_q:
                cand = self.swapped_q[0]
                need = self._get_block_needed(cand)
                if len(self.running_q) + 1 <= self.engine_config.max_batch_size and \
                        self.num_decoding_gpu_blocks + need <= self.num_gpu_blocks:
                    self.running_q.append(cand)
                    self.num_decoding_gpu_blocks += need
                    self.swapped_q.popleft()
                    returned.append(cand)
                    grow_budget = -1          # free blocks are about to be used: no give-back this call
                else:
                    break
        if cfg.quant_serve and grow_budget == cfg.num_layers_to_quantize:
            self.try_quant2org(engine)
        return self.running_q, returned, evicted

    def _admit_prefill(self, engine, grow_budget: int) -> Tuple[List[Request], int, int]:
        """Head-of-line admission of waiting prompts (scheduler.py:97-166).  Under
        ``quant_serve`` a prompt that does not fit may trigger pool growth: allowed while
        ``next_unquantized_layer >= num_layers_to_quantize_max``, the shortfall is within
        this call's budget and that many layers are left; the reference then spends the
        WHOLE remaining budget at once ("aggressive" replacement)."""
        cfg, ecfg = engine.engine_config, self.engine_config
        batch: List[Request] = []
        blocks = tokens = 0
        while self.waiting_q:
            req = self.waiting_q[0]
            need = self._get_block_needed(req)
            room = len(batch) + 1 <= ecfg.max_batch_size and \
                len(self.running_q) + len(batch) + 1 <= ecfg.max_batch_size and \
                tokens + req.prompt_len <= ecfg.max_tokens_in_batch
            if not room:
                break
            if cfg.quant_serve:
                short = self.segments_short(blocks + need, engine.model.kv_cache_new_block_size)
                if short > 0:
                    nxt = engine.model.next_unquantized_layer
                    if not (nxt >= cfg.num_layers_to_quantize_max and short <= grow_budget and nxt - short >= 0):
                        break
                    for _ in range(grow_budget):
                        self._grow(engine)
                    grow_budget = 0
            elif blocks + need + self.num_decoding_gpu_blocks > self.num_gpu_blocks:
                break
            batch.append(req)
            blocks += need
            tokens += req.prompt_len
            self.waiting_q.popleft()
        return batch, blocks, grow_budget

    def on_batch_finish(self, batch: List[Request]) -> None:
        self.request_id_manager.free_ids([r.request_id for r in batch if r.is_finished()])
        self.running_q = [r for r in self.running_q if not r.is_finished()]
