"""The two sublayers of a Kekapel layer, each a function from its normalised input to its raw output; the residual
bookkeeping around them (post-norm into the fp32 stream, the next input norm) is the model's fused step."""
import torch

from swiftllm_amd import _hip

from ..kernels.linear import linear
from ..kernels.moe import moe_experts, moe_route
from ..kernels.polynorm import polynorm
from ..kernels.window_attn import qknorm_and_store_kv, window_attention


def _project(a: torch.Tensor, w: torch.Tensor, skinny: bool) -> torch.Tensor:
    """a [T, in] @ w[out, in]^T. bf16 / f16: the framework's projection routing (hand-written weight-streaming GEMMs for
    decode-sized batches, the BLAS otherwise); fp32: the BLAS in true fp32."""
    if a.dtype == torch.float32:
        return torch.nn.functional.linear(a, w)
    if skinny and not getattr(w, "_swl_blas_only", False):
        try:
            return linear(a, w, True)
        except _hip.HipLibraryError as exc:
            # a projection shape the hand-written decode GEMMs are not specialised for (they say so with the "not supported"
            # code): this weight goes through the BLAS from here on; any other failure is a real one
            if "code -2" not in str(exc):
                raise
            w._swl_blas_only = True
    return linear(a, w, False)


class KekapelAttention:
    """q/k/v projection -> per-head q/k norm + KV store -> windowed, capped, head-mixed attention over the pool -> output
    projection."""

    def __init__(self, layer_config, weight, eps: float, skinny: bool, max_positions: int = 1 << 20):
        self.mixer, self.w, self.eps, self.skinny = layer_config.mixer, weight, eps, skinny
        self.max_positions = max_positions

    def forward(self, h: torch.Tensor, pool, pool_slice, block_table, tok_seq, tok_pos, tiles=None) -> torch.Tensor:
        qkv = _project(h, self.w.qkv, self.skinny)
        qknorm_and_store_kv(qkv, self.w.q_norm, self.w.k_norm, pool, pool_slice, block_table, tok_seq, tok_pos,
                            self.mixer, self.eps)
        if pool is None:    # memory profiling: the attention's output buffer without its reads
            attn = torch.zeros((h.shape[0], self.mixer.num_q_heads * self.mixer.value_dim), dtype=h.dtype, device=h.device)
        else:
            attn = window_attention(qkv, self.w.talk, pool, pool_slice, block_table, tok_seq, tok_pos, self.mixer, tiles,
                                    self.max_positions)
        return _project(attn, self.w.o, self.skinny)


class KekapelFeedForward:
    def __init__(self, layer_config, weight, eps: float, skinny: bool):
        self.mlp, self.w, self.eps, self.skinny = layer_config.mlp, weight, eps, skinny

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        if self.mlp.kind == "dense":
            z = _project(h, self.w.up, self.skinny)
            return _project(polynorm(z, self.w.act, self.eps), self.w.down, self.skinny)
        idx, wts = moe_route(h, self.w.router, self.w.router_b, self.mlp.top_k)
        return moe_experts(h, idx, wts, self.w.gate_up, self.w.down, self.mlp.limit)
