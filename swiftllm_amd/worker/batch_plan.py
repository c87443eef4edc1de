"""Host-side batch planning: everything `LlamaModel.forward` derives from its Python-list arguments
before touching the device. Pure numpy — unit-tested on CPU against the reference's arithmetic.

Reference: swiftllm/worker/model.py:268-324 (flattening, sequence lengths, start offsets, position
indices, the seq_block_size heuristic) and post_layer.py:24-29 (last-token indices).
"""
import dataclasses
import itertools
from typing import List, Sequence

import numpy as np


def select_seq_block_size(decoding_seq_lens: Sequence[int], num_kv_heads: int,
                          num_slots: int = 256, max_splits: int = 128) -> int:
    """Split-K width (tokens) of flash-decoding, sized for MI355X.

    The reference halves 2048 until `KVH * sum(len) / width >= 1024` programs exist (model.py:305-324:
    "1024 because ~128 SMs", one 1-warp program per q-head). Our phase-1 workgroup is 8 waves serving
    a whole kv-head group, one per CU, so the right launch is ~`num_slots` (= CU count, 256)
    workgroups in whole rounds, each with as many KV blocks as possible:

        width = KVH * sum(len) / num_slots        (tokens per workgroup for one full round)

    rounded up to 64 tokens. When that width already covers the longest sequence there is a single
    sequence block per sequence — phase 1 writes the output directly and phase 2 is never launched —
    and the width is rounded up to 256 so it (and a captured hipGraph) stays valid while the
    sequences grow. The width is a free internal choice: results are invariant up to fp32
    reassociation, which tests/test_gpu_kernels.py checks.
    """
    if len(decoding_seq_lens) == 0:
        return 2048
    total = sum(-(-n // 64) * 64 for n in decoding_seq_lens)
    longest = max(decoding_seq_lens)
    size = max(64, -(-(num_kv_heads * total) // (num_slots * 64)) * 64)
    if size >= longest:
        size = -(-size // 256) * 256
    while -(-longest // size) > max_splits:
        size *= 2
    return size


@dataclasses.dataclass
class BatchPlan:
    batch_size: int
    num_tokens: int
    num_prefill_seqs: int
    num_prefill_tokens: int
    max_prefill_len: int
    num_decoding_seqs: int
    max_decoding_len: int
    seq_block_size: int
    num_seq_blocks: int
    seq_lengths_list: List[int]
    # int32 arrays
    input_ids: np.ndarray               # [T]
    seq_ids: np.ndarray                 # [B]
    seq_lengths: np.ndarray             # [B]
    prefill_seq_lens: np.ndarray        # [Bp]
    prefill_start_locs_with_end: np.ndarray  # [Bp + 1]
    decoding_seq_lens: np.ndarray       # [Bd]
    position_indices: np.ndarray        # [T]
    last_token_indices: np.ndarray      # [B]
    # sequences of the caller's batch; batch_size - num_real_seqs trailing rows are inert padding (length 0) that rounds a
    # pure-decode batch up to its hipGraph bucket (worker/model.py: _decode_batch_bucket). -1: not set = batch_size
    num_real_seqs: int = -1

    @property
    def real_seqs(self) -> int:
        return self.num_real_seqs if self.num_real_seqs >= 0 else self.batch_size

    SEGMENTS = ("input_ids", "seq_ids", "seq_lengths", "prefill_seq_lens",
                "prefill_start_locs_with_end", "decoding_seq_lens", "position_indices",
                "last_token_indices")

    def packed_layout(self):
        """(name, offset, size) of every array inside one int32 buffer; offsets are multiples of 4
        elements (16 bytes). The layout depends only on (T, B, Bp), so a replayed hipGraph of a
        pure-decode batch of size B always finds its metadata at the same addresses."""
        out, off = [], 0
        for name in self.SEGMENTS:
            n = getattr(self, name).size
            out.append((name, off, n))
            off += (n + 3) // 4 * 4
        return out, off

    def pack_into(self, buf: np.ndarray) -> int:
        layout, total = self.packed_layout()
        for name, off, n in layout:
            buf[off:off + n] = getattr(self, name)
        return total


def plan_batch(input_ids_list: Sequence[Sequence[int]], seq_ids_list: Sequence[int],
               decoding_seq_lens_list: Sequence[int], num_kv_heads: int,
               num_slots: int = 256) -> BatchPlan:
    """Prefill sequences come first in all three lists (reference model.py:268-270); a decoding
    sequence contributes exactly one token and its length INCLUDES that token."""
    batch_size = len(input_ids_list)
    num_decoding = len(decoding_seq_lens_list)
    num_prefill = batch_size - num_decoding
    if num_prefill < 0 or len(seq_ids_list) != batch_size:
        raise ValueError("inconsistent batch: need len(seq_ids) == len(input_ids) >= len(decoding_seq_lens)")
    prefill_lens = [len(ids) for ids in input_ids_list[:num_prefill]]
    flat = np.fromiter(itertools.chain.from_iterable(input_ids_list), dtype=np.int32)
    num_tokens = flat.size
    num_prefill_tokens = sum(prefill_lens)
    if num_tokens - num_prefill_tokens != num_decoding:
        raise ValueError("every decoding sequence must contribute exactly one token")
    pl = np.asarray(prefill_lens, dtype=np.int32)
    dl = np.asarray(decoding_seq_lens_list, dtype=np.int32)
    starts_with_end = np.zeros(num_prefill + 1, dtype=np.int32)
    np.cumsum(pl, out=starts_with_end[1:])
    pos = np.empty(num_tokens, dtype=np.int32)
    if num_prefill_tokens:
        # 0..len-1 for every prefill sequence: global arange minus each token's sequence start
        pos[:num_prefill_tokens] = (np.arange(num_prefill_tokens, dtype=np.int32)
                                    - np.repeat(starts_with_end[:-1], pl))
    pos[num_prefill_tokens:] = dl - 1
    last = np.concatenate((starts_with_end[1:] - 1,
                           np.arange(num_prefill_tokens, num_tokens, dtype=np.int32))).astype(np.int32)
    sbs = select_seq_block_size(decoding_seq_lens_list, num_kv_heads, num_slots)
    max_dec = max(decoding_seq_lens_list) if num_decoding else 0
    seq_lengths_list = prefill_lens + list(decoding_seq_lens_list)
    return BatchPlan(
        batch_size=batch_size, num_tokens=num_tokens, num_prefill_seqs=num_prefill,
        num_prefill_tokens=num_prefill_tokens,
        max_prefill_len=max(prefill_lens) if prefill_lens else 0,
        num_decoding_seqs=num_decoding, max_decoding_len=max_dec, seq_block_size=sbs,
        num_seq_blocks=(max_dec + sbs - 1) // sbs, seq_lengths_list=seq_lengths_list,
        input_ids=flat, seq_ids=np.asarray(seq_ids_list, dtype=np.int32),
        seq_lengths=np.asarray(seq_lengths_list, dtype=np.int32), prefill_seq_lens=pl,
        prefill_start_locs_with_end=starts_with_end, decoding_seq_lens=dl, position_indices=pos,
        last_token_indices=last)


# ---- token-level steps: prompt portions and decoded tokens in one batch ----------------------------------------------------
@dataclasses.dataclass
class StepEntry:
    """The tokens one sequence brings to a step: `tokens` continue the sequence at position `start` (0 for a new sequence;
    a decoded token is a portion of length one). `want`: offsets inside `tokens` whose logits the caller asks for."""
    seq_id: int
    tokens: Sequence[int]
    start: int
    want: Sequence[int] = ()


@dataclasses.dataclass
class StepPlan:
    """Flat per-token metadata of a step. Kernels that serve portions and decoded tokens alike need nothing else: a token's
    block-table row, its position, and (for the output) which rows are asked for."""
    num_tokens: int
    num_seqs: int
    seq_ids_list: List[int]
    target_lens_list: List[int]         # length of every sequence after the step (what the block allocator must cover)
    input_ids: np.ndarray               # [T] int32
    tok_pos: np.ndarray                 # [T] int32 position of each token in its sequence
    tok_seq: np.ndarray                 # [T] int32 block-table row of each token
    want_rows: np.ndarray               # [R] int32 rows (into the T tokens) whose logits are produced
    # tiles of up to TILE consecutive tokens of one sequence (the matrix-core attention's unit of work)
    tile_row0: np.ndarray = None        # [NT] int32 first token row of each tile
    tile_cnt: np.ndarray = None         # [NT] int32 tokens in it
    # the portions themselves (what recurrent layers walk token by token) and, per token, where its portion starts
    seq_row0: np.ndarray = None         # [S] int32 first token row of each sequence's portion
    seq_cnt: np.ndarray = None          # [S] int32 tokens in it
    tok_start: np.ndarray = None        # [T] int32 position of the first token of the token's portion
    # [T] int32 state slot * 2 + tail parity of the token's sequence; zeros until a worker with per-sequence state fills it
    tok_state: np.ndarray = None

    TILE = 16
    SEGMENTS = ("input_ids", "tok_pos", "tok_seq", "want_rows", "tile_row0", "tile_cnt", "seq_row0", "seq_cnt", "tok_start",
                "tok_state")

    def packed_layout(self):
        out, off = [], 0
        for name in self.SEGMENTS:
            n = getattr(self, name).size
            out.append((name, off, n))
            off += (n + 3) // 4 * 4
        return out, off

    def pack_into(self, buf: np.ndarray) -> int:
        layout, total = self.packed_layout()
        for name, off, n in layout:
            buf[off:off + n] = getattr(self, name)
        return total


def plan_step(entries: Sequence[StepEntry], vocab_size: int = None, max_positions: int = None) -> StepPlan:
    """Flatten the entries in order. Checked here, on the host, so that nothing out of range reaches a kernel: token ids
    against the vocabulary, positions against the position table, one entry per sequence."""
    ids, pos, seq, want, seq_ids, targets = [], [], [], [], [], []
    base = 0
    for e in entries:
        n = len(e.tokens)
        if n == 0:
            raise ValueError(f"sequence {e.seq_id} brings no tokens to the step")
        if e.start < 0:
            raise ValueError(f"sequence {e.seq_id}: negative start {e.start}")
        if max_positions is not None and e.start + n > max_positions:
            raise RuntimeError(f"sequence {e.seq_id} would reach position {e.start + n - 1}, the model has "
                               f"{max_positions} positions")
        if e.seq_id in seq_ids:
            raise ValueError(f"sequence {e.seq_id} appears twice in one step")
        toks = np.asarray(e.tokens, dtype=np.int64)
        if vocab_size is not None and (toks.min() < 0 or toks.max() >= vocab_size):
            raise ValueError(f"sequence {e.seq_id}: token ids must be in [0, {vocab_size})")
        ids.append(toks.astype(np.int32))
        pos.append(np.arange(e.start, e.start + n, dtype=np.int32))
        seq.append(np.full(n, e.seq_id, dtype=np.int32))
        for w in e.want:
            if not 0 <= w < n:
                raise ValueError(f"sequence {e.seq_id}: wanted offset {w} outside its {n} tokens")
            want.append(base + w)
        seq_ids.append(int(e.seq_id))
        targets.append(int(e.start + n))
        base += n
    cat = (lambda xs: np.concatenate(xs) if xs else np.empty(0, dtype=np.int32))
    row0, cnt, at = [], [], 0
    for e in entries:
        n = len(e.tokens)
        starts = np.arange(0, n, StepPlan.TILE, dtype=np.int32)
        row0.append(at + starts)
        cnt.append(np.minimum(StepPlan.TILE, n - starts).astype(np.int32))
        at += n
    counts = np.asarray([len(e.tokens) for e in entries], dtype=np.int32)
    starts = np.asarray([e.start for e in entries], dtype=np.int32)
    return StepPlan(tile_row0=cat(row0), tile_cnt=cat(cnt), seq_cnt=counts,
                    seq_row0=(np.cumsum(counts) - counts).astype(np.int32), tok_start=np.repeat(starts, counts),
                    tok_state=np.zeros(base, dtype=np.int32),
                    num_tokens=base, num_seqs=len(seq_ids), seq_ids_list=seq_ids, target_lens_list=targets,
                    input_ids=cat(ids), tok_pos=cat(pos), tok_seq=cat(seq), want_rows=np.asarray(want, dtype=np.int32))
