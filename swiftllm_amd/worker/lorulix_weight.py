"""Weight containers and checkpoint reader for Lorulix.

Tensor names are the checkpoint's: `embed`, `pos`, `final.norm`, `head`, and per layer `l<i>.`: `norm1 / norm1b / norm2 /
norm2b`, `canon1 / canon2` ([width, taps]), `rg1 / rg2` (+ `.b`), the mixer's `mix.*` and the feed-forward's `mlp.*`.
Linear weights are [out, in].

What the loader does with them:
  * projection matrices go to the device in the compute dtype; matrices that multiply the same input are concatenated into
    one (attention: q | k | v; delta rule: q | k | v | output gate | beta | decay; dense feed-forward: gate | up; shared
    expert: up | its per-token gate), experts are stacked ([experts, ff, width], [experts, width, ff]);
  * everything that enters fp32 arithmetic — norm weights (stored around zero: kept as 1 + w), convolution taps (stored
    [channels, taps], kept tap-major [taps, channels] so that a lane reads the taps of 8 channels with two 16-byte loads),
    gate biases, q/k norm weights, the recurrence's A_log / dt_bias / output norm, the router — is kept in fp32 (exact: the
    checkpoint holds bfloat16);
  * the learned distance bias [rows, heads] is expanded once, on the host in float64, to a table [heads, positions] indexed
    by distance, so that no kernel evaluates the bucket function.
Shapes are checked against config.json before anything is used.
"""
from typing import List

import torch

from swiftllm_amd.model_config import distance_bias_rows

from .kekapel_weight import Getter, _checkpoint_getter


class LorulixLayerWeight:
    def __init__(self, layer_id: int):
        self.layer_id = layer_id

    def load(self, get: Getter, cfg, lcfg, dtype, device):
        w, mx, p = cfg.hidden_size, lcfg.mixer, f"l{self.layer_id}."

        def f32(name, shape):
            return get(p + name, shape).to(device=device, dtype=torch.float32).contiguous()

        def one_plus(name, shape):
            return (1.0 + get(p + name, shape).to(torch.float32)).to(device).contiguous()

        def mat(name, shape):
            return get(p + name, shape).to(device=device, dtype=dtype).contiguous()

        for k in ("1", "2") if lcfg.mlp is not None else ("1",):
            setattr(self, "norm" + k, one_plus("norm" + k, (w,)))
            setattr(self, "norm" + k + "b", one_plus("norm" + k + "b", (w,)))
            setattr(self, "canon" + k, f32("canon" + k, (w, cfg.canon_taps)).t().contiguous())      # tap-major
            setattr(self, "rg" + k, mat("rg" + k, (w, w)))
            setattr(self, "rg" + k + "_b", f32("rg" + k + ".b", (w,)))
        if lcfg.type == "attention":
            q = mat("mix.q", (mx.q_size, w))
            self.q_norm = f32("mix.q.norm", (mx.q_size,))
            if mx.kv_from < 0:
                self.qkv = torch.cat((q, mat("mix.k", (mx.k_size, w)), mat("mix.v", (mx.v_size, w))), dim=0).contiguous()
                self.k_norm = f32("mix.k.norm", (mx.k_size,))
            else:
                self.qkv, self.k_norm = q, None
            self.rel = None
            if mx.bias_max > 0:
                table = get(p + "mix.rel", (None, mx.num_q_heads)).to(torch.float32)     # (the row count is the tensor's)
                row_of = torch.tensor(distance_bias_rows(table.shape[0], mx.bias_max, cfg.max_position_embeddings))
                self.rel = table[row_of].t().contiguous().to(device)      # [heads, positions] by distance
            self.o = mat("mix.o", (w, mx.num_q_heads * mx.value_dim))
        else:
            H, t = mx.num_heads, mx.conv_taps
            self.proj = torch.cat((mat("mix.q", (mx.qk_size, w)), mat("mix.k", (mx.qk_size, w)),
                                   mat("mix.v", (mx.v_size, w)), mat("mix.g", (mx.v_size, w)), mat("mix.b", (H, w)),
                                   mat("mix.a", (H, w))), dim=0).contiguous()
            self.conv = torch.cat((f32("mix.q.conv", (mx.qk_size, t)), f32("mix.k.conv", (mx.qk_size, t)),
                                   f32("mix.v.conv", (mx.v_size, t))), dim=0).t().contiguous()     # tap-major
            self.a_log = f32("mix.A_log", (H,))
            self.dt_bias = f32("mix.dt_bias", (H,))
            self.out_norm = f32("mix.norm", (mx.value_dim,))
            self.o = mat("mix.o", (w, mx.v_size))
        mlp = lcfg.mlp
        if mlp is None:
            return
        ff = mlp.ffn_inter_dim
        if mlp.kind == "dense":
            self.gate_up = torch.cat((mat("mlp.gate", (ff, w)), mat("mlp.up", (ff, w))), dim=0).contiguous()
            self.down = mat("mlp.down", (w, ff))
        else:
            self.router = f32("mlp.router", (mlp.num_experts, w))
            self.up = torch.empty((mlp.num_experts, ff, w), dtype=dtype, device=device)
            self.down = torch.empty((mlp.num_experts, w, ff), dtype=dtype, device=device)
            for e in range(mlp.num_experts):
                self.up[e] = mat(f"mlp.e{e}.up", (ff, w))
                self.down[e] = mat(f"mlp.e{e}.down", (w, ff))
            self.shared_up = self.shared_down = None
            if mlp.shared_ffn_inter_dim:
                fs = mlp.shared_ffn_inter_dim
                self.shared_up = torch.cat((mat("mlp.shared.up", (fs, w)), mat("mlp.shared.sg", (1, w))), dim=0).contiguous()
                self.shared_down = mat("mlp.shared.down", (w, fs))


class LorulixWeight:
    def __init__(self, model_config, dtype: torch.dtype):
        self.model_config = model_config
        self.dtype = dtype
        self.layers = [LorulixLayerWeight(i) for i in range(model_config.num_layers)]

    def load(self, get: Getter, device):
        cfg, dtype = self.model_config, self.dtype
        w = cfg.hidden_size
        self.embed = get("embed", (cfg.vocab_size, w)).to(device=device, dtype=dtype).contiguous()
        self.pos = get("pos", (cfg.max_position_embeddings, w)).to(device=device, dtype=dtype).contiguous()
        self.final_norm = (1.0 + get("final.norm", (w,)).to(torch.float32)).to(device).contiguous()
        self.head = get("head", (cfg.vocab_size, w)).to(device=device, dtype=dtype).contiguous()
        for layer, lcfg in zip(self.layers, cfg.layers):
            layer.load(get, cfg, lcfg, dtype, device)

    def projection_tensors(self) -> List[torch.Tensor]:
        """The 2-D matrices a step multiplies through `linear` (candidates for the decode GEMMs' packed copies)."""
        out = [self.head]
        for layer in self.layers:
            for a in ("rg1", "rg2", "qkv", "proj", "o", "gate_up", "shared_up", "shared_down"):
                t = getattr(layer, a, None)
                if t is not None:
                    out.append(t)
            if getattr(layer, "down", None) is not None and layer.down.dim() == 2:
                out.append(layer.down)
        return out


DUMMY_BIAS_ROWS = 32


def _dummy_getter(seed: int = 0) -> Getter:
    """Random weights of the checkpoint's shapes (benchmarks, memory profiling): matrices ~ N(0, 1/in), weights stored
    around zero and biases small — a stream that stays finite through any depth."""
    g = torch.Generator().manual_seed(seed)

    def get(name: str, shape: tuple) -> torch.Tensor:
        leaf = name.split(".")[-1]
        if leaf == "rel":
            return 0.5 * torch.randn((DUMMY_BIAS_ROWS, shape[1]), generator=g)
        if leaf == "conv" or "canon" in leaf:
            return torch.randn(shape, generator=g) / shape[1]
        if leaf in ("A_log", "dt_bias"):
            return 0.5 * torch.randn(shape, generator=g)
        if len(shape) == 2:
            return torch.randn(shape, generator=g) / shape[1] ** 0.5
        if leaf == "norm" and name.endswith("mix.norm"):
            return 1.0 + 0.02 * torch.randn(shape, generator=g)
        if name.endswith("q.norm") or name.endswith("k.norm"):
            return 1.0 + 0.02 * torch.randn(shape, generator=g)
        return 0.02 * torch.randn(shape, generator=g)
    return get


def load_lorulix_weights(model_config, dtype: torch.dtype, model_path: str, use_dummy: bool = False,
                         device="cuda") -> LorulixWeight:
    weight = LorulixWeight(model_config, dtype)
    get = _dummy_getter() if use_dummy else _checkpoint_getter(model_path)
    weight.load(get, torch.device(device))
    return weight
