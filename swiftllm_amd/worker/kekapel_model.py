"""KekapelModel — the data-plane worker for the Kekapel design.

The worker protocol, the token-level `step`, the block pool, the block managers, hipGraph replay of decode steps and
swapping are SteppedModel's (stepped_model.py); this file adds what is Kekapel's: the layout of a block (a 16-token block
holds, side by side, the keys and values of every LAYER RUN — a layer inside the loop runs several times with the same
weights and has a separate slice per pass), the weights, and the stack: embedding, sandwich LayerNorms fused with the fp32
stream update, attention and feed-forward sublayers, the loop's pass additions. Projections run in the compute dtype
(bfloat16 / float16, or true float32).
"""
from typing import List

import torch

from swiftllm_amd.engine_config import EngineConfig
from swiftllm_amd.model_config import KekapelModelConfig

from .kekapel_weight import load_kekapel_weights
from .kernels.layernorm import add_layernorm, embed_positions, layernorm
from .kernels.linear import pack_weight, packable
from .kernels.window_attn import PoolSlice
from .layers.kekapel_layer import KekapelAttention, KekapelFeedForward, _project
from .stepped_model import SteppedModel


class _Sublayer:
    """One residual update of the stack: x += mult * LN_post(f(LN_pre(x)))."""
    __slots__ = ("kind", "run", "op", "pre", "post", "pass_index", "ends_run")


class KekapelModel(SteppedModel):
    CONFIG_CLASS = KekapelModelConfig

    @torch.inference_mode()
    def __init__(self, engine_config: EngineConfig):
        self.sublayers: List[_Sublayer] = []
        self.pool_slices: List[PoolSlice] = []
        super().__init__(engine_config)

    def _layout_pool(self):
        """Offsets (in elements) of every layer run's keys and values inside a block."""
        cfg, bs = self.model_config, self.engine_config.block_size
        off = 0
        self.pool_slices = []
        for run in cfg.layer_runs:
            mx = cfg.layers[run.layer].mixer
            k_off = off
            off += mx.k_size * bs
            self.pool_slices.append(PoolSlice(k_off, off))
            off += mx.v_size * bs
        self.block_elems = off

    def _build(self):
        cfg, ecfg = self.model_config, self.engine_config
        self.weight = load_kekapel_weights(cfg, self.dtype, ecfg.model_path, ecfg.use_dummy, self.device)
        skinny = bool(getattr(ecfg, "use_skinny_gemm", False)) and self.dtype != torch.float32
        if skinny and getattr(ecfg, "pack_decode_weights", False):
            for t in self.weight.projection_tensors():
                if packable(t):
                    pack_weight(t)
        self._skinny = skinny
        eps = cfg.norm_eps
        self.sublayers = []
        for run in cfg.layer_runs:
            lcfg, lw = cfg.layers[run.layer], self.weight.layers[run.layer]
            s = _Sublayer()
            s.kind, s.run, s.op = "mixer", run.index, KekapelAttention(lcfg, lw, eps, skinny, cfg.max_position_embeddings)
            s.pre, s.post, s.pass_index = (lw.norm1_w, lw.norm1_b), (lw.norm1b_w, lw.norm1b_b), run.pass_index
            s.ends_run = lcfg.mlp is None
            self.sublayers.append(s)
            if lcfg.mlp is not None:
                f = _Sublayer()
                f.kind, f.run, f.op = "ff", run.index, KekapelFeedForward(lcfg, lw, eps, skinny)
                f.pre, f.post, f.pass_index, f.ends_run = (lw.norm2_w, lw.norm2_b), (lw.norm2b_w, lw.norm2b_b), -1, True
                self.sublayers.append(f)

    @torch.inference_mode()
    def _run_stack(self, dev: dict, use_pool: bool) -> torch.Tensor:
        """Embedding -> every sublayer -> the fp32 stream [T, width]."""
        cfg, w = self.model_config, self.weight
        eps, mult = cfg.norm_eps, cfg.residual_mult
        pool = self.kv_pool if use_pool else None
        block_table = self.gpu_block_manager.block_table if use_pool else None
        x, x0 = embed_positions(dev["input_ids"], dev["tok_pos"], w.embed, w.pos, cfg.embedding_scale,
                                keep_copy=cfg.loop_times > 1)
        tap = self.layer_tap
        subs = self.sublayers

        def pass_adds(s):
            """What is added to the stream right before sublayer s: (embedding output or None, step vector or None)."""
            if s is None or s.pass_index < 0:
                return None, None
            return (x0 if s.pass_index > 0 else None), w.loop_step[s.pass_index]

        a0, st = pass_adds(subs[0])
        h = add_layernorm(x, None, mult, None, a0, st, subs[0].pre, eps, self.dtype)
        for i, s in enumerate(subs):
            if s.kind == "mixer":
                y = s.op.forward(h, pool, self.pool_slices[s.run] if use_pool else None, block_table, dev["tok_seq"],
                                 dev["tok_pos"], (dev["tile_row0"], dev["tile_cnt"]))
            else:
                y = s.op.forward(h)
            nxt = subs[i + 1] if i + 1 < len(subs) else None
            a0, st = pass_adds(nxt)
            if tap is not None and s.ends_run:
                # unfused, so that the stream can be read between the layer's last update and the next pass's additions
                add_layernorm(x, y, mult, s.post, eps=eps)
                tap.append(x.clone())
                h = add_layernorm(x, None, mult, None, a0, st, nxt.pre, eps, self.dtype) if nxt is not None else None
            else:
                h = add_layernorm(x, y, mult, s.post, a0, st, nxt.pre if nxt is not None else None, eps, self.dtype)
        return x

    @torch.inference_mode()
    def _logits(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        """Final norm of the asked-for rows and the vocabulary projection -> [rows, vocab] in the compute dtype."""
        w = self.weight
        h = layernorm(x, w.final_norm_w, w.final_norm_b, self.model_config.norm_eps, self.dtype, rows)
        return _project(h, w.head, self._skinny)
