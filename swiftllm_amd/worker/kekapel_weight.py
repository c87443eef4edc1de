"""Weight containers and checkpoint reader for Kekapel.

Tensor names are the checkpoint's: `embed`, `pos`, `loop.step`, `final.norm(.b)`, `head`, and per layer `l<i>.`:
`norm1 / norm1b / norm2 / norm2b` (+ `.b`), `mix.q / k / v / o`, `mix.q.norm`, `mix.k.norm`, `mix.talk`, and either
`mlp.up / down / act` or `mlp.router(.b)` + `mlp.e<j>.gate / up / down`. Linear weights are [out, in].

What the loader does with them:
  * projection matrices go to the device in the compute dtype; q, k and v are concatenated into one `qkv` matrix (one GEMM
    per mixer), an expert's gate and up rows into `gate_up`, and the experts are stacked ([experts, 2 ff, width],
    [experts, width, ff]) so that the expert kernels index them by expert id;
  * everything that enters fp32 arithmetic — norm weights and biases, the q/k norm weights, the head-mixing matrix, the
    router and its bias, the loop step vectors — is kept in fp32 (exact: the checkpoint holds bfloat16);
  * the four PolyNorm coefficients become Python floats (kernel arguments).
Shapes are checked against config.json before anything is used.
"""
import os
from typing import Callable, List

import torch

from .weight import _read_safetensors_index

Getter = Callable[[str, tuple], torch.Tensor]


class KekapelLayerWeight:
    def __init__(self, layer_id: int):
        self.layer_id = layer_id

    def load(self, get: Getter, cfg, lcfg, dtype, device):
        w, mx, p = cfg.hidden_size, lcfg.mixer, f"l{self.layer_id}."

        def f32(name, shape):
            return get(p + name, shape).to(device=device, dtype=torch.float32).contiguous()

        def mat(name, shape):
            return get(p + name, shape).to(device=device, dtype=dtype).contiguous()

        names = ("norm1", "norm1b") + (("norm2", "norm2b") if lcfg.mlp is not None else ())
        for nm in names:
            setattr(self, nm + "_w", f32(nm, (w,)))
            setattr(self, nm + "_b", f32(nm + ".b", (w,)))
        self.qkv = torch.cat((mat("mix.q", (mx.q_size, w)), mat("mix.k", (mx.k_size, w)), mat("mix.v", (mx.v_size, w))),
                             dim=0).contiguous()
        self.q_norm = f32("mix.q.norm", (mx.head_dim,))
        self.k_norm = f32("mix.k.norm", (mx.head_dim,))
        self.talk = f32("mix.talk", (mx.num_q_heads, mx.num_q_heads))
        self.o = mat("mix.o", (w, mx.num_q_heads * mx.value_dim))
        mlp = lcfg.mlp
        if mlp is None:
            return
        ff = mlp.ffn_inter_dim
        if mlp.kind == "dense":
            self.up = mat("mlp.up", (ff, w))
            self.down = mat("mlp.down", (w, ff))
            self.act = [float(x) for x in get(p + "mlp.act", (4,)).float().tolist()]
        else:
            self.router = f32("mlp.router", (mlp.num_experts, w))
            self.router_b = f32("mlp.router.b", (mlp.num_experts,))
            self.gate_up = torch.empty((mlp.num_experts, 2 * ff, w), dtype=dtype, device=device)
            self.down = torch.empty((mlp.num_experts, w, ff), dtype=dtype, device=device)
            for e in range(mlp.num_experts):
                self.gate_up[e, :ff] = mat(f"mlp.e{e}.gate", (ff, w))
                self.gate_up[e, ff:] = mat(f"mlp.e{e}.up", (ff, w))
                self.down[e] = mat(f"mlp.e{e}.down", (w, ff))


class KekapelWeight:
    def __init__(self, model_config, dtype: torch.dtype):
        self.model_config = model_config
        self.dtype = dtype
        self.layers = [KekapelLayerWeight(i) for i in range(model_config.num_layers)]

    def load(self, get: Getter, device):
        cfg, dtype = self.model_config, self.dtype
        w = cfg.hidden_size
        self.embed = get("embed", (cfg.vocab_size, w)).to(device=device, dtype=dtype).contiguous()
        self.pos = get("pos", (cfg.max_position_embeddings, w)).to(device=device, dtype=dtype).contiguous()
        self.loop_step = None
        if cfg.loop_times:
            self.loop_step = get("loop.step", (cfg.loop_times, w)).to(device=device, dtype=torch.float32).contiguous()
        self.final_norm_w = get("final.norm", (w,)).to(device=device, dtype=torch.float32).contiguous()
        self.final_norm_b = get("final.norm.b", (w,)).to(device=device, dtype=torch.float32).contiguous()
        self.head = get("head", (cfg.vocab_size, w)).to(device=device, dtype=dtype).contiguous()
        for layer, lcfg in zip(self.layers, cfg.layers):
            layer.load(get, cfg, lcfg, dtype, device)

    def projection_tensors(self) -> List[torch.Tensor]:
        """The 2-D matrices a step multiplies through `linear` (candidates for the decode GEMMs' packed copies)."""
        out = [self.head]
        for layer in self.layers:
            out += [getattr(layer, a) for a in ("qkv", "o", "up") if hasattr(layer, a)]
            if hasattr(layer, "down") and layer.down.dim() == 2:
                out.append(layer.down)
        return out


def _checkpoint_getter(model_path: str) -> Getter:
    """Tensors straight from the safetensors files: header parsed here, data memory-mapped, nothing executed."""
    import numpy as np
    files = sorted(n for n in os.listdir(model_path) if n.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors file in {model_path}")
    table = _read_safetensors_index(model_path, files)
    maps = {}
    kinds = {"BF16": (torch.bfloat16, 2), "F16": (torch.float16, 2), "F32": (torch.float32, 4), "I32": (torch.int32, 4)}

    def get(name: str, shape: tuple) -> torch.Tensor:
        if name not in table:
            raise KeyError(f"weight {name} not found in the checkpoint")
        path, st_dtype, st_shape, b, e = table[name]
        if len(st_shape) != len(shape) or any(b is not None and a != b for a, b in zip(st_shape, shape)):     # None: any size
            raise ValueError(f"shape of weight {name} does not match: {tuple(st_shape)} vs {tuple(shape)}")
        if st_dtype not in kinds:
            raise TypeError(f"weight {name}: unsupported dtype {st_dtype}")
        tdtype, size = kinds[st_dtype]
        if path not in maps:
            maps[path] = np.memmap(path, dtype=np.uint8, mode="r")
        raw = torch.from_numpy(np.array(maps[path][b:e], copy=True))
        return raw.view(tdtype).reshape(tuple(st_shape))
    return get


def _dummy_getter(seed: int = 0) -> Getter:
    """Random weights of the checkpoint's shapes (benchmarks, memory profiling): matrices ~ N(0, 1/in), norm weights
    near one, biases near zero — a stream that stays finite through any depth."""
    g = torch.Generator().manual_seed(seed)

    def get(name: str, shape: tuple) -> torch.Tensor:
        leaf = name.split(".")[-1]
        if name.endswith("mix.talk"):
            return torch.eye(shape[0]) + 0.1 * torch.randn(shape, generator=g)
        if name.endswith(".act"):
            return torch.tensor([0.6, 0.3, 0.1, 0.0])
        if len(shape) == 2:
            return torch.randn(shape, generator=g) / shape[1] ** 0.5
        if leaf == "b":
            return 0.02 * torch.randn(shape, generator=g)
        return 1.0 + 0.02 * torch.randn(shape, generator=g)
    return get


def load_kekapel_weights(model_config, dtype: torch.dtype, model_path: str, use_dummy: bool = False,
                         device="cuda") -> KekapelWeight:
    weight = KekapelWeight(model_config, dtype)
    get = _dummy_getter() if use_dummy else _checkpoint_getter(model_path)
    weight.load(get, torch.device(device))
    return weight
