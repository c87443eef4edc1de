"""SteppedModel — the worker that every design with a token-level step shares.

A design's worker (KekapelModel, LorulixModel) supplies its configuration class, the layout of a block of the pool, its
weights and the stack itself (`_run_stack`, `_logits`); everything around the stack lives here and is the same for all of
them:

    model = Model(engine_config); model.load_weights()
    n = model.profile_num_blocks(); model.init_kvcache_and_swap(n)
    tokens = model.forward(input_ids_list, seq_ids_list, decoding_seq_lens_list)       # the worker protocol
    logits = model.step(entries)                                                       # portions + decoded tokens
    model.swap_in_seqs(ids) / model.swap_out_seqs(ids) / model.free_seqs_resources(ids)

State: ONE block pool [num_blocks, elements per block] in the compute dtype, managed by the framework's BlockManager (block
table, allocator, swapping), and — for designs with recurrent layers — a StateSlotManager (`self.state`): one fp32 slot per
running sequence. `step` plans the batch on the host (worker/batch_plan.py), brings the block table and the state slots up
to date, uploads the plan through one pinned buffer and runs the stack; pure-decode steps replay a captured hipGraph.
"""
import math
from typing import List, Sequence

import numpy as np
import torch

from swiftllm_amd import _hip
from swiftllm_amd.engine_config import EngineConfig
from swiftllm_amd.utils import GB

from .batch_plan import StepEntry, StepPlan, plan_step
from .block_manager import BlockManager
from .kernels.block_swapping import swap_blocks
from .kernels.sampling import argmax_rows

DTYPES = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float32": torch.float32}


class SteppedModel:
    SUPPORTED_DTYPES = tuple(DTYPES)
    CONFIG_CLASS = None         # the design's configuration class (model_config.py)

    @torch.inference_mode()
    def __init__(self, engine_config: EngineConfig):
        self.engine_config = engine_config
        self.model_config = self.CONFIG_CLASS.load_from_model_path(engine_config.model_path)
        self.dtype = DTYPES[getattr(engine_config, "dtype", "bfloat16")]
        self.device = torch.device("cuda")
        self.weight = None
        self.num_blocks = None
        self.kv_pool = self.kv_swap = None
        self.gpu_block_manager = self.cpu_block_manager = None
        self.state = None           # StateSlotManager of designs with per-sequence recurrent state
        self.block_elems = 0
        self._layout_pool()
        self._meta_host = self._meta_host_np = self._meta_dev = self._meta_done = None
        self.after_launch_hook = None
        # pure-decode steps (every sequence brings one token and asks for its logits) replay a captured hipGraph, one per
        # batch size: the step's launch geometry depends on the token count only, never on positions, block ids or slots
        self._decode_graphs = {}
        self._graph_pool = None
        self.graph_captures = 0
        # tests set these to lists: the fp32 stream after every layer run / the logits of every step
        self.layer_tap = None
        self.logits_tap = None
        # what the scheduler asks any worker: how long a sequence may grow
        self.max_seq_len = self.model_config.max_position_embeddings

    # ---- what a design supplies ----------------------------------------------------------------------------------------------
    def _layout_pool(self):
        """Set self.block_elems (and the design's own offsets inside a block)."""
        raise NotImplementedError

    def _build(self):
        """Load self.weight and build the stack (called by load_weights on the device)."""
        raise NotImplementedError

    def _run_stack(self, dev: dict, use_pool: bool) -> torch.Tensor:
        """Embedding -> every sublayer -> the fp32 stream [T, width]."""
        raise NotImplementedError

    def _logits(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    # ---- set-up ------------------------------------------------------------------------------------------------------
    @torch.inference_mode()
    def load_weights(self):
        if not torch.cuda.is_available():
            raise _hip.HipLibraryError("no HIP device visible: swiftllm_amd's data plane runs only on an AMD GPU (gfx950)")
        _hip.load()
        if self.dtype == torch.float32:
            torch.backends.cuda.matmul.allow_tf32 = False      # true fp32 products
            torch.set_float32_matmul_precision("highest")
        self._build()

    @torch.inference_mode()
    def profile_num_blocks(self) -> int:
        """How many blocks fit: one forged worst-case step without a pool, the allocator's high-water mark, and the rest
        of the usable memory divided by a block's bytes."""
        ecfg = self.engine_config
        torch.cuda.empty_cache()
        torch.cuda.reset_peak_memory_stats()
        num_tokens = min(ecfg.max_tokens_in_batch, ecfg.max_batch_size * self.model_config.max_position_embeddings)
        batch = min(ecfg.max_batch_size, num_tokens)
        lens = [num_tokens // batch] * batch
        lens[-1] += num_tokens % batch
        saved = self.kv_pool
        self.kv_pool = None
        self.forward([[0] * n for n in lens], list(range(batch)), [], ignore_kvcache=True)
        if self.state is not None:
            self.state.release(list(range(batch)))
        self.kv_pool = saved
        torch.cuda.synchronize()
        free_memory, total_memory = torch.cuda.mem_get_info()
        peak = total_memory - free_memory
        usable = total_memory * ecfg.gpu_mem_utilization
        print(f"[Model.profile] GPU total memory: {total_memory / GB:.2f} GB, runtime peak memory: {peak / GB:.2f} GB")
        if usable < peak:
            raise RuntimeError(f"Peak memory {peak / GB:.2f} GB exceeds usable memory {usable / GB:.2f} GB")
        block_bytes = self.block_elems * self.dtype.itemsize
        table_bytes = 2 * ecfg.max_seqs_in_block_table * ecfg.max_blocks_per_seq * 4
        torch.cuda.empty_cache()
        return max(math.floor((usable - peak - table_bytes) / block_bytes), 0)

    @torch.inference_mode()
    def init_kvcache_and_swap(self, num_blocks: int):
        ecfg = self.engine_config
        self.num_blocks = num_blocks
        # zeros: a slot that was never written must not hold NaN bit patterns
        self.kv_pool = torch.zeros((num_blocks, self.block_elems), dtype=self.dtype, device=self.device)
        pin = getattr(ecfg, "pin_swap_memory", True) and ecfg.num_cpu_blocks > 0
        try:
            self.kv_swap = torch.zeros((ecfg.num_cpu_blocks, self.block_elems), dtype=self.dtype, pin_memory=pin)
        except RuntimeError:
            self.kv_swap = torch.zeros((ecfg.num_cpu_blocks, self.block_elems), dtype=self.dtype)
        self._decode_graphs.clear()     # (captured against the previous pool and block table)
        self._graph_pool = None
        self.gpu_block_manager = BlockManager("GPU", num_blocks, ecfg.max_seqs_in_block_table, ecfg.max_blocks_per_seq,
                                              ecfg.block_size, self.device)
        self.cpu_block_manager = BlockManager("CPU", ecfg.num_cpu_blocks, ecfg.max_seqs_in_block_table,
                                              ecfg.max_blocks_per_seq, ecfg.block_size, self.device)

    # ---- one step ----------------------------------------------------------------------------------------------------
    def _upload_plan(self, plan: StepPlan):
        """The plan's int32 arrays through ONE pinned buffer and ONE async copy; returns device views."""
        layout, total = plan.packed_layout()
        if self._meta_done is not None:
            self._meta_done.synchronize()
        if self._meta_host is None or self._meta_host.numel() < total:
            cap = max(total, 4 * self.engine_config.max_tokens_in_batch + 64)
            self._meta_host = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self._meta_host_np = self._meta_host.numpy()
            self._meta_dev = torch.empty(cap, dtype=torch.int32, device=self.device)
            self._meta_done = torch.cuda.Event()
        plan.pack_into(self._meta_host_np)
        self._meta_dev[:total].copy_(self._meta_host[:total], non_blocking=True)
        self._meta_done.record()
        return {name: self._meta_dev[off:off + n] for name, off, n in layout}

    def _begin_state_step(self, plan: StepPlan):
        """Per-sequence state: slots for the sequences of this step, their codes into the plan."""
        if self.state is None:
            return
        starts = [int(plan.tok_pos[r]) for r in plan.seq_row0]
        codes = self.state.begin_step(plan.seq_ids_list, starts)
        plan.tok_state = np.repeat(codes, plan.seq_cnt).astype(np.int32)

    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry], ignore_kvcache: bool = False) -> torch.Tensor:
        """Run one batch of portions. Returns the logits of the wanted places, [wanted, vocab] (device tensor in the compute
        dtype), in the order of the entries and of each entry's `want`."""
        cfg = self.model_config
        plan = plan_step(entries, cfg.vocab_size, cfg.max_position_embeddings)
        if plan.num_tokens == 0:
            return torch.empty((0, cfg.vocab_size), dtype=self.dtype, device=self.device)
        if not ignore_kvcache:
            self.gpu_block_manager.allocate_blocks_for_seqs(plan.seq_ids_list, plan.target_lens_list)
        self._begin_state_step(plan)
        dev = self._upload_plan(plan)
        if (getattr(self.engine_config, "use_hip_graph", False) and not ignore_kvcache and self.layer_tap is None
                and plan.num_tokens == plan.num_seqs == plan.want_rows.size):
            logits = self._step_decode_graph(plan, dev)
        else:
            x = self._run_stack(dev, not ignore_kvcache)
            if plan.want_rows.size == 0:
                return torch.empty((0, cfg.vocab_size), dtype=self.dtype, device=self.device)
            logits = self._logits(x, dev["want_rows"])
        if self.logits_tap is not None:
            self.logits_tap.append(logits.clone())
        return logits

    _MAX_DECODE_GRAPHS = 64

    def _step_decode_graph(self, plan: StepPlan, dev: dict) -> torch.Tensor:
        """Replay (capturing it first, once per batch size) the whole pure-decode step. The metadata buffer has a fixed
        address and a layout that depends on the token count only, so a replay reads this step's tokens, positions and
        block-table rows from where the capture did. The returned logits are the graph's own output buffer: valid until
        the next replay of the same graph."""
        key = plan.num_tokens
        entry = self._decode_graphs.pop(key, None)
        if entry is not None and entry[2] != self._meta_dev.data_ptr():
            entry = None        # the metadata buffer was re-allocated: the capture points at the old one
        if entry is None:
            self.graph_captures += 1
            # one eager run first: nothing may be lazily initialised under capture. The replay below runs the step once more:
            # writes into the block pool repeat themselves, recurrent state does not, so its slots are put back
            saved = self.state.snapshot(plan.seq_ids_list) if self.state is not None else None
            warm = torch.cuda.Stream()
            warm.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(warm):
                self._logits(self._run_stack(dev, True), dev["want_rows"])
            torch.cuda.current_stream().wait_stream(warm)
            if saved is not None:
                self.state.restore(saved)
            while len(self._decode_graphs) >= self._MAX_DECODE_GRAPHS:
                self._decode_graphs.pop(next(iter(self._decode_graphs)))
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                out = self._logits(self._run_stack(dev, True), dev["want_rows"])
            entry = (graph, out, self._meta_dev.data_ptr())
        self._decode_graphs[key] = entry
        entry[0].replay()
        return entry[1]

    @torch.inference_mode()
    def forward(self, input_ids_list: List[List[int]], seq_ids_list: List[int], decoding_seq_lens_list: List[int],
                ignore_kvcache: bool = False) -> List[int]:
        """The worker protocol's iteration: whole prompts first, then decoding sequences (one token each, their lengths
        INCLUDING it). Returns the greedy next token of every sequence."""
        if len(input_ids_list) == 0:
            return []
        num_prefill = len(input_ids_list) - len(decoding_seq_lens_list)
        if num_prefill < 0 or len(seq_ids_list) != len(input_ids_list):
            raise ValueError("inconsistent batch: need len(seq_ids) == len(input_ids) >= len(decoding_seq_lens)")
        entries = []
        for i, (ids, sid) in enumerate(zip(input_ids_list, seq_ids_list)):
            if i < num_prefill:
                entries.append(StepEntry(sid, ids, 0, (len(ids) - 1,)))
            else:
                if len(ids) != 1:
                    raise ValueError("every decoding sequence must contribute exactly one token")
                entries.append(StepEntry(sid, ids, decoding_seq_lens_list[i - num_prefill] - 1, (0,)))
        logits = self.step(entries, ignore_kvcache)
        tokens = argmax_rows(logits)
        if self.after_launch_hook is not None:
            self.after_launch_hook()
        return tokens.tolist()

    # ---- swapping / release ------------------------------------------------------------------------------------------
    def _swap(self, seq_ids_list: List[int], is_swap_in: bool):
        if len(seq_ids_list) == 0:
            return
        src_mgr = self.cpu_block_manager if is_swap_in else self.gpu_block_manager
        dst_mgr = self.gpu_block_manager if is_swap_in else self.cpu_block_manager
        counts = src_mgr.get_num_allocated_blocks_host(seq_ids_list)
        src_ids = [b for s in seq_ids_list for b in src_mgr.get_block_ids_host(s)]
        src_mgr.gather_allocated_blocks_and_free(seq_ids_list)
        dst_mgr.allocate_blocks_for_seqs(seq_ids_list, [c * self.engine_config.block_size for c in counts])
        dst_ids = [b for s in seq_ids_list for b in dst_mgr.get_block_ids_host(s)]
        swap_blocks(src_ids, dst_ids, is_swap_in, self.kv_pool, None, self.kv_swap, None)
        if self.state is not None:
            (self.state.swap_in if is_swap_in else self.state.swap_out)(seq_ids_list)

    @torch.inference_mode()
    def swap_in_seqs(self, seq_ids_list: List[int]):
        self._swap(seq_ids_list, True)

    @torch.inference_mode()
    def swap_out_seqs(self, seq_ids_list: List[int]):
        self._swap(seq_ids_list, False)

    @torch.inference_mode()
    def free_seqs_resources(self, seq_ids_list: List[int]):
        if len(seq_ids_list) == 0:
            return
        self.gpu_block_manager.free_blocks_for_seqs(seq_ids_list)
        self.cpu_block_manager.free_blocks_for_seqs(seq_ids_list)
        if self.state is not None:
            self.state.release(seq_ids_list)
