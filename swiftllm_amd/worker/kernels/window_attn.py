"""Attention over the paged pool for models whose heads are coupled before the softmax: per-head q/k RMS norm fused with
the KV store, then sliding-window attention with tanh soft-capping and an [H, H] head-mixing matrix. Prompt portions (with
or without a cached prefix) and decoded tokens go through the same two launches: every token carries its block-table row
and its position. csrc/qknorm_kv.hip, csrc/window_attn.hip."""
import torch

from swiftllm_amd import _hip


class PoolSlice:
    """Where one layer run keeps its keys and values inside the shared block pool: element offsets inside a block."""
    __slots__ = ("k_offset", "v_offset")

    def __init__(self, k_offset: int, v_offset: int):
        self.k_offset, self.v_offset = k_offset, v_offset


def qknorm_and_store_kv(qkv: torch.Tensor, q_norm: torch.Tensor, k_norm: torch.Tensor, pool: torch.Tensor,
                        pool_slice: PoolSlice, block_table: torch.Tensor, tok_seq: torch.Tensor, tok_pos: torch.Tensor,
                        mixer, eps: float):
    """qkv [T, q | k | v] of one fused projection: q heads normalised in place, k heads normalised into the pool, v heads
    copied into the pool. pool None (memory profiling): only the query norm."""
    _hip.require_gpu_tensor(qkv, "qkv")
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == mixer.q_size + mixer.k_size + mixer.v_size
    assert q_norm.dtype == k_norm.dtype == torch.float32 and q_norm.numel() == k_norm.numel() == mixer.head_dim
    assert tok_pos.dtype == torch.int32 and tok_pos.shape[0] == qkv.shape[0]
    kp = vp = 0
    stride = 0
    if pool is not None:
        assert pool.is_contiguous() and pool.dtype == qkv.dtype and block_table.is_contiguous()
        assert tok_seq.dtype == torch.int32 and tok_seq.shape[0] == qkv.shape[0]
        esize = pool.element_size()
        kp = pool.data_ptr() + pool_slice.k_offset * esize
        vp = pool.data_ptr() + pool_slice.v_offset * esize
        stride = pool.shape[1]
    _hip.call("swl_qknorm_store_kv", _hip.ptr(qkv), _hip.ptr(q_norm), _hip.ptr(k_norm), kp, vp, _hip.ptr(block_table),
              _hip.ptr(tok_seq), _hip.ptr(tok_pos), qkv.shape[0], mixer.num_q_heads, mixer.num_kv_heads, mixer.head_dim,
              mixer.value_dim, qkv.stride(0), block_table.shape[1] if block_table is not None else 0, stride, float(eps),
              _hip.dtype_code3(qkv.dtype), _hip.stream())


def qknorm_full_and_store_kv(q_or_qkv: torch.Tensor, q_norm: torch.Tensor, k_norm: torch.Tensor, pool: torch.Tensor,
                             pool_slice: PoolSlice, block_table: torch.Tensor, tok_seq: torch.Tensor,
                             tok_pos: torch.Tensor, mixer, eps: float, store: bool):
    """Whole-projection RMS norms (a weight per element) with the position-dependent query multiplier of `mixer`
    (q_temp_coef, q_temp_every). store: the rows are [q | k | v] and k, v go to the pool; else the rows are queries only."""
    _hip.require_gpu_tensor(q_or_qkv, "qkv")
    width = mixer.q_size + ((mixer.k_size + mixer.v_size) if store else 0)
    assert q_or_qkv.dim() == 2 and q_or_qkv.stride(1) == 1 and q_or_qkv.shape[1] == width
    assert q_norm.dtype == torch.float32 and q_norm.numel() == mixer.q_size
    assert tok_pos.dtype == torch.int32 and tok_pos.shape[0] == q_or_qkv.shape[0]
    kp = vp = stride = 0
    if store and pool is not None:
        assert k_norm.dtype == torch.float32 and k_norm.numel() == mixer.k_size
        assert pool.is_contiguous() and pool.dtype == q_or_qkv.dtype and block_table.is_contiguous()
        esize = pool.element_size()
        kp = pool.data_ptr() + pool_slice.k_offset * esize
        vp = pool.data_ptr() + pool_slice.v_offset * esize
        stride = pool.shape[1]
    _hip.call("swl_qknorm_full_store_kv", _hip.ptr(q_or_qkv), _hip.ptr(q_norm), _hip.ptr(k_norm), kp, vp,
              _hip.ptr(block_table), _hip.ptr(tok_seq), _hip.ptr(tok_pos), q_or_qkv.shape[0], mixer.num_q_heads,
              mixer.num_kv_heads, mixer.head_dim, mixer.value_dim, q_or_qkv.stride(0),
              block_table.shape[1] if block_table is not None else 0, stride, float(eps), float(mixer.q_temp_coef),
              int(mixer.q_temp_every), _hip.dtype_code3(q_or_qkv.dtype), _hip.stream())


# Steps with at least this many tokens go to the matrix-core kernel (tiles of up to 16 queries; a decoded token is a tile of
# one: the matrix core is mostly padding there, but the kernel reads every page once with wide loads and shares a tile's pages
# out over several workgroups when there are few tiles).
TILES_MIN_TOKENS = 1
_NUM_CUS = 256
_scratch = {}       # device -> persistent fp32 scratch of the key-split partials (fixed address: hipGraph replays use it)
_retired = []


def _split_scratch(device, floats: int) -> torch.Tensor:
    buf = _scratch.get(device)
    if buf is None or buf.numel() < floats:
        if buf is not None:
            _retired.append(buf)        # a captured graph may still replay against it
        buf = torch.empty(max(floats, 1 << 20), dtype=torch.float32, device=device)
        _scratch[device] = buf
    return buf


def choose_key_splits(num_tiles: int, mixer, max_positions: int) -> int:
    """Workgroups per tile: enough to occupy the chip when a step has few tiles, never more than the pages a tile can see.
    A function of the tile count and the model only (not of positions), so a captured decode graph stays valid."""
    span = mixer.window if mixer.window > 0 else max_positions
    pages = span // 16 + 2
    return max(1, min(_NUM_CUS // max(num_tiles, 1), pages // 4, 16))


def tiles_supported(mixer, dtype: torch.dtype) -> bool:
    if dtype not in (torch.float16, torch.bfloat16):
        return False
    return bool(_hip.load().swl_window_attn_tiles_supported(mixer.num_q_heads, mixer.num_kv_heads, mixer.head_dim,
                                                            mixer.value_dim, _hip.dtype_code(dtype)))


def window_attention(qkv: torch.Tensor, talk: torch.Tensor, pool: torch.Tensor, pool_slice: PoolSlice,
                     block_table: torch.Tensor, tok_seq: torch.Tensor, tok_pos: torch.Tensor, mixer,
                     tiles=None, max_positions: int = 1 << 20, rel: torch.Tensor = None) -> torch.Tensor:
    """-> [T, heads * vdim]. The queries are the (already normalised) first columns of qkv; keys and values come from the
    pool, which already holds this step's tokens. `tiles` = (tile_row0, tile_cnt) device arrays: the step cut into runs of
    up to 16 consecutive tokens of one sequence — given, and the shape served, the matrix-core kernel runs. `talk` None: the
    heads are not mixed. `rel` (fp32 [heads, distances]): a bias added to head h's score at distance query - key."""
    _hip.require_gpu_tensor(qkv, "qkv")
    assert talk is None or (talk.dtype == torch.float32 and talk.is_contiguous()
                            and talk.shape == (mixer.num_q_heads, mixer.num_q_heads))
    assert rel is None or (rel.dtype == torch.float32 and rel.is_contiguous() and rel.shape[0] == mixer.num_q_heads)
    rel_len = rel.shape[1] if rel is not None else 0
    assert pool.is_contiguous() and pool.dtype == qkv.dtype
    n = qkv.shape[0]
    out = torch.empty((n, mixer.num_q_heads * mixer.value_dim), dtype=qkv.dtype, device=qkv.device)
    esize = pool.element_size()
    if tiles is not None and n >= TILES_MIN_TOKENS and tiles_supported(mixer, qkv.dtype):
        row0, cnt = tiles
        splits = choose_key_splits(row0.shape[0], mixer, max_positions)
        scratch = None
        if splits > 1:
            scratch = _split_scratch(qkv.device, splits * n * mixer.num_q_heads * (mixer.value_dim + 2))
        _hip.call("swl_window_attn_tiles", _hip.ptr(out), _hip.ptr(qkv), pool.data_ptr() + pool_slice.k_offset * esize,
                  pool.data_ptr() + pool_slice.v_offset * esize, _hip.ptr(block_table), _hip.ptr(tok_seq),
                  _hip.ptr(tok_pos), _hip.ptr(row0), _hip.ptr(cnt), _hip.ptr(talk), _hip.ptr(rel), rel_len, row0.shape[0],
                  mixer.num_q_heads,
                  mixer.num_kv_heads, mixer.head_dim, mixer.value_dim, qkv.stride(0), mixer.window, float(mixer.scale),
                  float(mixer.softcap), block_table.shape[1], pool.shape[1], splits, _hip.ptr(scratch), n,
                  _hip.dtype_code(qkv.dtype), _hip.stream())
        return out
    _hip.call("swl_window_attn", _hip.ptr(out), _hip.ptr(qkv), pool.data_ptr() + pool_slice.k_offset * esize,
              pool.data_ptr() + pool_slice.v_offset * esize, _hip.ptr(block_table), _hip.ptr(tok_seq), _hip.ptr(tok_pos),
              _hip.ptr(talk), _hip.ptr(rel), rel_len, n, mixer.num_q_heads, mixer.num_kv_heads, mixer.head_dim,
              mixer.value_dim, qkv.stride(0),
              mixer.window, float(mixer.scale), float(mixer.softcap), block_table.shape[1], pool.shape[1],
              _hip.dtype_code3(qkv.dtype), _hip.stream())
    return out
