"""The gated delta rule as a recurrent mixer with per-sequence state slots. csrc/delta_rule.hip."""
import torch

from swiftllm_amd import _hip

from .rms_stream import StateRef


def delta_rule_mixer(proj: torch.Tensor, conv_w: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
                     norm_w: torch.Tensor, st: StateRef, tail_off: int, state_off: int, mixer, eps: float) -> torch.Tensor:
    """proj [T, q | k | v | gate | b | a] (one fused projection) -> [T, heads * vdim] in proj's dtype: short convolutions
    (conv_w tap-major [taps, q | k | v channels]) +
    SiLU, unit q / k, the token-by-token recurrence on the fp32 state [heads, dim, vdim] at `state_off` inside each
    sequence's slot, then per head o / rms(o) * norm_w * silu(gate)."""
    _hip.require_gpu_tensor(proj, "proj")
    n = proj.shape[0]
    H, G, d, dv = mixer.num_heads, mixer.num_kv_heads, mixer.head_dim, mixer.value_dim
    assert proj.stride(1) == 1 and proj.shape[1] == mixer.proj_size
    assert conv_w.dtype == torch.float32 and conv_w.is_contiguous() and conv_w.shape == (mixer.conv_taps, mixer.conv_channels)
    assert a_log.dtype == dt_bias.dtype == norm_w.dtype == torch.float32 and a_log.numel() == dt_bias.numel() == H
    assert norm_w.numel() == dv
    dev, f32 = proj.device, torch.float32
    qn = torch.empty((n, G * d), dtype=f32, device=dev)
    kn = torch.empty((n, G * d), dtype=f32, device=dev)
    kq = torch.empty((n, G), dtype=f32, device=dev)
    vv = torch.empty((n, H * dv), dtype=f32, device=dev)
    beta = torch.empty((n, H), dtype=f32, device=dev)
    decay = torch.empty((n, H), dtype=f32, device=dev)
    code, stream = _hip.dtype_code3(proj.dtype), _hip.stream()
    _hip.call("swl_delta_prep", _hip.ptr(qn), _hip.ptr(kn), _hip.ptr(kq), _hip.ptr(vv), _hip.ptr(beta), _hip.ptr(decay), _hip.ptr(proj),
              proj.stride(0), _hip.ptr(conv_w), _hip.ptr(a_log), _hip.ptr(dt_bias), _hip.ptr(st.pool), st.pool.stride(0),
              int(tail_off), _hip.ptr(st.tok_pos), _hip.ptr(st.tok_start), _hip.ptr(st.tok_state), _hip.ptr(st.tok_seq), n,
              H, G, d, dv, mixer.conv_taps, code, stream)
    o = torch.empty((n, H * dv), dtype=f32, device=dev)
    _hip.call("swl_delta_rule", _hip.ptr(o), _hip.ptr(qn), _hip.ptr(kn), _hip.ptr(kq), _hip.ptr(vv), _hip.ptr(beta), _hip.ptr(decay),
              _hip.ptr(st.pool), st.pool.stride(0), int(state_off), _hip.ptr(st.seq_row0), _hip.ptr(st.seq_cnt),
              _hip.ptr(st.tok_pos), _hip.ptr(st.tok_state), st.seq_row0.shape[0], H, G, d, dv, stream)
    out = torch.empty((n, H * dv), dtype=proj.dtype, device=dev)
    gate = proj[:, mixer.conv_channels:mixer.conv_channels + H * dv]
    _hip.call("swl_gated_head_rmsnorm", _hip.ptr(out), _hip.ptr(o), _hip.ptr(gate), proj.stride(0), _hip.ptr(norm_w),
              float(eps), n, H, dv, code, stream)
    return out
