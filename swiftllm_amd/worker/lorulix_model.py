"""LorulixModel — the data-plane worker for the Lorulix design.

The worker protocol, the token-level `step`, the block pool, the block managers, hipGraph replay of decode steps and
swapping are SteppedModel's (stepped_model.py); this file adds what is Lorulix's:

  * the layout of a block: the keys and values of every attention layer that has its own (a layer that borrows another
    layer's reads that layer's slice);
  * the layout of a state slot (StateSlotManager): per sublayer the carried inputs of its input convolution, per delta-rule
    layer the carried inputs of its q/k/v convolutions and the fp32 state [heads, dim, vdim];
  * the stack: embedding with learned positions, then per sublayer
        r  = W_rg h + (bias in the step)            gate logits, from the normed stream h
        hc = h + conv(h)                            causal input convolution with carried state
        m  = sublayer(hc)
        x += norm_b(m * sigmoid(r));  h = norm(x)   one fused launch between two sublayers (kernels/rms_stream.py)
    with the stream x in fp32 and projections in the compute dtype (bfloat16 / float16, or true float32).
"""
from typing import List

import torch

from swiftllm_amd.engine_config import EngineConfig
from swiftllm_amd.model_config import LorulixModelConfig

from .kernels.layernorm import embed_positions
from .kernels.linear import pack_weight, packable
from .kernels.rms_stream import StateRef, causal_conv_state, gated_add_rmsnorm
from .kernels.window_attn import PoolSlice
from .layers.kekapel_layer import _project
from .layers.lorulix_layer import LorulixAttention, LorulixDelta, LorulixFeedForward, StepContext
from .lorulix_weight import load_lorulix_weights
from .state_slots import StateSlotManager
from .stepped_model import SteppedModel


class _Sublayer:
    """One residual update of the stack: x += norm_post(f(h + conv(h)) * sigmoid(W_rg h + b)), h = norm_pre(x)."""
    __slots__ = ("op", "pre", "post", "canon", "canon_off", "rg", "rg_b", "ends_layer")


class LorulixModel(SteppedModel):
    CONFIG_CLASS = LorulixModelConfig

    @torch.inference_mode()
    def __init__(self, engine_config: EngineConfig):
        self.sublayers: List[_Sublayer] = []
        self.pool_slices = {}
        super().__init__(engine_config)

    def _layout_pool(self):
        """Offsets (in elements) of every attention layer's own keys and values inside a block."""
        cfg, bs = self.model_config, self.engine_config.block_size
        off = 0
        self.pool_slices = {}
        for i, layer in enumerate(cfg.layers):
            if layer.type == "attention" and layer.mixer.kv_from < 0:
                k_off = off
                off += layer.mixer.k_size * bs
                self.pool_slices[i] = PoolSlice(k_off, off)
                off += layer.mixer.v_size * bs
        for i, layer in enumerate(cfg.layers):
            if layer.type == "attention" and layer.mixer.kv_from >= 0:
                self.pool_slices[i] = self.pool_slices[layer.mixer.kv_from]
        self.block_elems = max(off, 8)      # (a model without attention layers still has a block table)

    def _build(self):
        cfg, ecfg = self.model_config, self.engine_config
        self.weight = load_lorulix_weights(cfg, self.dtype, ecfg.model_path, ecfg.use_dummy, self.device)
        skinny = bool(getattr(ecfg, "use_skinny_gemm", False)) and self.dtype != torch.float32
        if skinny and getattr(ecfg, "pack_decode_weights", False):
            for t in self.weight.projection_tensors():
                if packable(t):
                    pack_weight(t)
        self._skinny = skinny
        eps, w, taps = cfg.norm_eps, cfg.hidden_size, cfg.canon_taps
        # one slot per sequence that runs: as many as a batch holds
        self.state = StateSlotManager(ecfg.max_batch_size, self.device)
        self.sublayers = []
        for i, (lcfg, lw) in enumerate(zip(cfg.layers, self.weight.layers)):
            mx = lcfg.mixer
            s = _Sublayer()
            if lcfg.type == "attention":
                s.op = LorulixAttention(lcfg, lw, eps, skinny, self.pool_slices[i], cfg.max_position_embeddings)
            else:
                tail_off = self.state.add_region(2 * (mx.conv_taps - 1) * mx.conv_channels)
                state_off = self.state.add_region(mx.state_elems)
                s.op = LorulixDelta(lcfg, lw, eps, skinny, tail_off, state_off)
            s.pre, s.post, s.canon, s.rg, s.rg_b = lw.norm1, lw.norm1b, lw.canon1, lw.rg1, lw.rg1_b
            s.canon_off = self.state.add_region(2 * (taps - 1) * w)
            s.ends_layer = lcfg.mlp is None
            self.sublayers.append(s)
            if lcfg.mlp is not None:
                f = _Sublayer()
                f.op = LorulixFeedForward(lcfg, lw, skinny)
                f.pre, f.post, f.canon, f.rg, f.rg_b = lw.norm2, lw.norm2b, lw.canon2, lw.rg2, lw.rg2_b
                f.canon_off = self.state.add_region(2 * (taps - 1) * w)
                f.ends_layer = True
                self.sublayers.append(f)
        self.state.allocate()

    @torch.inference_mode()
    def _run_stack(self, dev: dict, use_pool: bool) -> torch.Tensor:
        """Embedding -> every sublayer -> the fp32 stream [T, width]."""
        cfg, w = self.model_config, self.weight
        eps = cfg.norm_eps
        st = StateRef(self.state.pool, dev["tok_pos"], dev["tok_start"], dev["tok_state"], dev["tok_seq"], dev["seq_row0"],
                      dev["seq_cnt"])
        ctx = StepContext(self.kv_pool if use_pool else None, self.gpu_block_manager.block_table if use_pool else None,
                          dev["tok_seq"], dev["tok_pos"], (dev["tile_row0"], dev["tile_cnt"]), st)
        x, _ = embed_positions(dev["input_ids"], dev["tok_pos"], w.embed, w.pos, 1.0, keep_copy=False)
        tap = self.layer_tap
        subs = self.sublayers
        h = gated_add_rmsnorm(x, pre=subs[0].pre, eps=eps, out_dtype=self.dtype)
        for i, s in enumerate(subs):
            r = _project(h, s.rg, self._skinny)
            hc = causal_conv_state(h, s.canon, st, s.canon_off, add_input=True)
            m, m2, m2_gate = s.op.forward(hc, ctx)
            nxt = subs[i + 1].pre if i + 1 < len(subs) else None
            h = gated_add_rmsnorm(x, m, s.post, r, s.rg_b, m2, m2_gate, pre=nxt, eps=eps)
            if tap is not None and s.ends_layer:
                tap.append(x.clone())
        return x

    @torch.inference_mode()
    def _logits(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        """The model's norm of the asked-for rows and the vocabulary projection -> [rows, vocab] in the compute dtype."""
        h = gated_add_rmsnorm(x, pre=self.weight.final_norm, eps=self.model_config.norm_eps, out_dtype=self.dtype,
                              row_idx=rows)
        return _project(h, self.weight.head, self._skinny)
