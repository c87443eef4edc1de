"""PolyNorm activation: a N(z) + b N(z^2) + c N(z^3) + e with N = division by the row's root mean square (fp32
statistics). csrc/polynorm.hip."""
import torch

from swiftllm_amd import _hip


def polynorm(z: torch.Tensor, coeffs, eps: float) -> torch.Tensor:
    _hip.require_gpu_tensor(z, "z")
    assert z.dim() == 2 and z.is_contiguous() and len(coeffs) == 4
    out = torch.empty_like(z)
    a, b, c, e = (float(v) for v in coeffs)
    _hip.call("swl_polynorm", _hip.ptr(out), _hip.ptr(z), a, b, c, e, float(eps), z.shape[0], z.shape[1],
              _hip.dtype_code3(z.dtype), _hip.stream())
    return out
