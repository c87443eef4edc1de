"""A plain, slow Lorulix for the tests: one function per mechanism, whole sequences, float64, dense masks, token loops.

Nothing here is shared with swiftllm_amd: the product computes the same design with a paged cache, state slots and HIP
kernels, this file with full [tokens, tokens] score matrices and Python loops over tokens. `W` is a dict name -> tensor
with the checkpoint's tensor names, `cfg` the parsed config.json.

Notation: n tokens, positions 0..n-1; H query heads, G key/value heads, d the query/key size, e the value size.
"""
import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return unit_rms(x, eps) * (1.0 + w)


def causal_conv(h, w):
    """h [n, C], w [C, taps]: out[t] = sum_j w[:, j] * h[t - taps + 1 + j], zeros before the first token. The last column
    multiplies the current token."""
    n, taps = h.shape[0], w.shape[1]
    out = torch.zeros_like(h)
    for j in range(taps):
        back = taps - 1 - j
        if back < n:
            out[back:] += w[:, j] * h[:n - back]
    return out


def silu(z):
    return z * torch.sigmoid(z)


# ---- gated delta rule ------------------------------------------------------------------------------------------------------
def delta_scan(q, k, v, beta, g, state=None):
    """One head. q, k [n, d] (already unit vectors, q scaled), v [n, e], beta, g [n]. state [d, e] or None (zeros).
    Per token: decay the state, write the correction of what it predicts for k, read with q. -> (o [n, e], state)."""
    n, d = q.shape
    e = v.shape[1]
    S = torch.zeros(d, e, dtype=F64) if state is None else state.clone()
    o = torch.zeros(n, e, dtype=F64)
    for t in range(n):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o, S


def delta_from_projections(qp, kp, vp, gp, bp, ap, W, pre, mx, eps):
    """Raw projections (q, k [n, G * d], v, gate [n, H * e], b, a [n, H]) -> the mixer's output before W_o, [n, H * e]."""
    n = qp.shape[0]
    H, G, d, e = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = silu(causal_conv(qp, W[pre + "q.conv"])).view(n, G, d)
    k = silu(causal_conv(kp, W[pre + "k.conv"])).view(n, G, d)
    v = silu(causal_conv(vp, W[pre + "v.conv"])).view(n, H, e)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(bp)
    decay = torch.exp(-torch.exp(W[pre + "A_log"]) * torch.nn.functional.softplus(ap + W[pre + "dt_bias"]))
    gate = silu(gp).view(n, H, e)
    out = torch.zeros(n, H, e, dtype=F64)
    for hd in range(H):
        kv = hd // (H // G)
        o, _ = delta_scan(q[:, kv], k[:, kv], v[:, hd], beta[:, hd], decay[:, hd])
        out[:, hd] = unit_rms(o, eps) * W[pre + "norm"] * gate[:, hd]
    return out.reshape(n, H * e)


def delta_mixer(h, W, pre, mx, eps):
    parts = [h @ W[pre + name].T for name in ("q", "k", "v", "g", "b", "a")]
    return delta_from_projections(*parts, W, pre, mx, eps) @ W[pre + "o"].T


# ---- attention with a learned distance bias -------------------------------------------------------------------------------
def distance_bucket(dist, rows, far):
    """Row of the bias table for a distance >= 0: one row per distance below rows // 2, logarithmic steps up to `far`."""
    half = rows // 2
    if dist < half:
        return dist
    return min(rows - 1, half + int(math.floor(math.log(dist / half) / math.log(far / half) * (rows - half))))


def query_temperature(n, coef, every):
    p = torch.arange(n, dtype=F64)
    return 1.0 + coef * torch.log(torch.floor((p + 1) / every) + 1.0)


def attention_keys_values(h, W, pre, mx, eps):
    """What a layer's cache holds: keys after their norm, values. [n, G, d], [n, G, e]."""
    n = h.shape[0]
    G, d, e = mx["kv_heads"], mx["dim"], mx["vdim"]
    k = unit_rms(h @ W[pre + "k"].T, eps) * W[pre + "k.norm"]
    v = h @ W[pre + "v"].T
    return k.view(n, G, d), v.view(n, G, e)


def attention_output(q, k, v, mx, rel=None):
    """q [n, H, d] (normed, with its temperature), k [n, G, d], v [n, G, e], rel [rows, H] or None -> [n, H * e]: softmax over
    every key j <= i of q_i . k_j * scale + rel[bucket(i - j)]."""
    n, H, G = q.shape[0], mx["heads"], mx["kv_heads"]
    k = k.repeat_interleave(H // G, dim=1)
    v = v.repeat_interleave(H // G, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, k) * mx["scale"]
    if rel is not None:
        row_of = torch.tensor([distance_bucket(dist, rel.shape[0], mx["bias_max"]) for dist in range(n)])
        dist = (torch.arange(n).unsqueeze(1) - torch.arange(n).unsqueeze(0)).clamp(min=0)
        s = s + rel[row_of[dist]].permute(2, 0, 1)
    i = torch.arange(n).unsqueeze(1)
    j = torch.arange(n).unsqueeze(0)
    s = s.masked_fill(j > i, float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("hij,jhd->ihd", p, v).reshape(n, -1)


def normed_queries(qp, qn, mx, eps):
    """qp [n, H * d] raw projection -> [n, H, d]: one RMS norm over the whole projection, then the temperature."""
    q = unit_rms(qp, eps) * qn
    temp = mx.get("q_temp")
    if temp:
        q = q * query_temperature(qp.shape[0], temp["coef"], temp["every"]).unsqueeze(1)
    return q.view(qp.shape[0], mx["heads"], mx["dim"])


def attention_mixer(h, W, pre, mx, eps, kv=None):
    """kv: (keys, values) of the layer this one borrows from, or None: its own."""
    q = normed_queries(h @ W[pre + "q"].T, W[pre + "q.norm"], mx, eps)
    k, v = attention_keys_values(h, W, pre, mx, eps) if kv is None else kv
    return attention_output(q, k, v, mx, W.get(pre + "rel")) @ W[pre + "o"].T


# ---- feed-forwards ----------------------------------------------------------------------------------------------------------
def dense_ff(h, W, pre, mlp):
    lim = mlp["limit"]
    g = torch.clamp(h @ W[pre + "gate"].T, max=lim)
    u = torch.clamp(h @ W[pre + "up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[pre + "down"].T


def relu_squared_expert(h, up, down):
    return torch.relu(h @ up.T) ** 2 @ down.T


def moe_ff(h, W, pre, mlp):
    E, top, scale = mlp["router"]["experts"], mlp["router"]["top"], mlp["router"]["scale"]
    s = torch.softmax(h @ W[pre + "router"].T, dim=-1)
    wts, idx = torch.topk(s, top, dim=-1)
    out = torch.zeros(h.shape[0], W[pre + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for j in range(top):
            ex = int(idx[t, j])
            out[t] += scale * wts[t, j] * relu_squared_expert(h[t:t + 1], W[f"{pre}e{ex}.up"], W[f"{pre}e{ex}.down"])[0]
    if mlp.get("shared"):
        sh = relu_squared_expert(h, W[pre + "shared.up"], W[pre + "shared.down"])
        out = out + torch.sigmoid(h @ W[pre + "shared.sg"].T) * sh
    return out


# ---- the stack ------------------------------------------------------------------------------------------------------------
def sublayer_input(h, W, name):
    """What a sublayer reads (the normed stream plus its causal convolution) and the gate on its result."""
    gate = torch.sigmoid(h @ W[name["rg"]].T + W[name["rg"] + ".b"])
    return h + causal_conv(h, W[name["canon"]]), gate


def forward(cfg, W, tokens, taps=None):
    """-> (logits [n, vocab], [the stream after every layer])."""
    W = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    n = len(tokens)
    x = W["embed"][torch.tensor(tokens)] + W["pos"][:n]
    streams, cache = [], {}
    for i, layer in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", layer["mixer"]
        h = norm_one_plus(x, W[p + "norm1"], eps)
        hc, gate = sublayer_input(h, W, {"rg": p + "rg1", "canon": p + "canon1"})
        if layer["type"] == "delta":
            m = delta_mixer(hc, W, p + "mix.", mx, eps)
        elif layer["type"] == "attention":
            src = mx.get("kv_from")
            if src is None:
                cache[i] = attention_keys_values(hc, W, p + "mix.", mx, eps)
            m = attention_mixer(hc, W, p + "mix.", mx, eps, cache[i if src is None else src])
        else:
            raise ValueError(layer["type"])
        x = x + norm_one_plus(m * gate, W[p + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp:
            h = norm_one_plus(x, W[p + "norm2"], eps)
            hc, gate = sublayer_input(h, W, {"rg": p + "rg2", "canon": p + "canon2"})
            f = dense_ff(hc, W, p + "mlp.", mlp) if mlp["kind"] == "dense" else moe_ff(hc, W, p + "mlp.", mlp)
            x = x + norm_one_plus(f * gate, W[p + "norm2b"], eps)
        streams.append(x.clone())
    logits = norm_one_plus(x, W["final.norm"], eps) @ W["head"].T
    return logits, streams


# ---- small configurations and random weights for the tests ----------------------------------------------------------------
def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, scale=0.3, bias_max=40, temp=(0.4, 8), kv_from=None, mlp=None):
    mixer = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "scale": scale, "vdim": vdim}
    if bias_max:
        mixer["bias_max"] = bias_max
    if temp:
        mixer["q_temp"] = {"coef": temp[0], "every": temp[1]}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def delta_layer(heads=4, kv_heads=2, dim=16, vdim=16, conv=4, mlp=None):
    return {"type": "delta", "mixer": {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim},
            "mlp": mlp}


def dense_mlp(ff, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe_mlp(ff, experts, top, scale=2.0, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


def make_config(width=48, vocab=96, layers=None, taps=3, max_positions=256, eps=1e-5):
    if layers is None:
        layers = [attention_layer(mlp=dense_mlp(80)), delta_layer(mlp=moe_mlp(32, 6, 2, shared=40)),
                  attention_layer(kv_from=0, mlp=moe_mlp(32, 4, 1))]
    return {"architecture": "Lorulix", "canon": {"taps": taps}, "layers": layers, "max_positions": max_positions,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def make_weights(cfg, seed=0, bias_rows=12):
    """Random bfloat16-representable weights with the checkpoint's names; sizes chosen so that every mechanism matters
    (gates away from saturation, decays neither 0 nor 1, a distance bias of the size of the scores)."""
    g = torch.Generator().manual_seed(seed)
    w = cfg["width"]
    taps = cfg["canon"]["taps"]

    def rnd(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)

    W = {"embed": rnd(cfg["vocab"], w), "pos": rnd(cfg["max_positions"], w, s=0.5), "final.norm": rnd(w, s=0.1),
         "head": rnd(cfg["vocab"], w, s=w ** -0.5)}
    for i, layer in enumerate(cfg["layers"]):
        p, mx, mlp = f"l{i}.", layer["mixer"], layer.get("mlp")
        for k in ("1", "2") if mlp else ("1",):
            W[p + "norm" + k] = rnd(w, s=0.1)
            W[p + "norm" + k + "b"] = rnd(w, s=0.1)
            W[p + "canon" + k] = rnd(w, taps, s=0.4)
            W[p + "rg" + k] = rnd(w, w, s=w ** -0.5)
            W[p + "rg" + k + ".b"] = rnd(w, s=0.5)
        H, G, d, e = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        if layer["type"] == "attention":
            W[p + "mix.q"] = rnd(H * d, w, s=w ** -0.5)
            W[p + "mix.q.norm"] = (1.0 + 0.2 * torch.randn(H * d, generator=g)).to(torch.bfloat16)
            if mx.get("kv_from") is None:
                W[p + "mix.k"] = rnd(G * d, w, s=w ** -0.5)
                W[p + "mix.v"] = rnd(G * e, w, s=w ** -0.5)
                W[p + "mix.k.norm"] = (1.0 + 0.2 * torch.randn(G * d, generator=g)).to(torch.bfloat16)
            if mx.get("bias_max"):
                W[p + "mix.rel"] = rnd(bias_rows, H, s=1.5)
            W[p + "mix.o"] = rnd(w, H * e, s=(H * e) ** -0.5)
        else:
            c = mx["conv"]
            W[p + "mix.q"], W[p + "mix.q.conv"] = rnd(G * d, w, s=w ** -0.5), rnd(G * d, c, s=0.6)
            W[p + "mix.k"], W[p + "mix.k.conv"] = rnd(G * d, w, s=w ** -0.5), rnd(G * d, c, s=0.6)
            W[p + "mix.v"], W[p + "mix.v.conv"] = rnd(H * e, w, s=w ** -0.5), rnd(H * e, c, s=0.6)
            W[p + "mix.b"], W[p + "mix.a"] = rnd(H, w, s=w ** -0.5), rnd(H, w, s=w ** -0.5)
            W[p + "mix.A_log"], W[p + "mix.dt_bias"] = rnd(H, s=0.5), rnd(H, s=0.5)
            W[p + "mix.norm"] = (1.0 + 0.2 * torch.randn(e, generator=g)).to(torch.bfloat16)
            W[p + "mix.g"] = rnd(H * e, w, s=w ** -0.5)
            W[p + "mix.o"] = rnd(w, H * e, s=(H * e) ** -0.5)
        if not mlp:
            continue
        if mlp["kind"] == "dense":
            ff = mlp["ff"]
            W[p + "mlp.gate"], W[p + "mlp.up"] = rnd(ff, w, s=2 * w ** -0.5), rnd(ff, w, s=2 * w ** -0.5)
            W[p + "mlp.down"] = rnd(w, ff, s=ff ** -0.5)
        else:
            ff = mlp["expert"]["ff"]
            W[p + "mlp.router"] = rnd(mlp["router"]["experts"], w, s=2 * w ** -0.5)
            for x in range(mlp["router"]["experts"]):
                W[f"{p}mlp.e{x}.up"] = rnd(ff, w, s=w ** -0.5)
                W[f"{p}mlp.e{x}.down"] = rnd(w, ff, s=ff ** -0.5)
            if mlp.get("shared"):
                fs = mlp["shared"]["ff"]
                W[p + "mlp.shared.up"], W[p + "mlp.shared.down"] = rnd(fs, w, s=w ** -0.5), rnd(w, fs, s=fs ** -0.5)
                W[p + "mlp.shared.sg"] = rnd(1, w, s=w ** -0.5)
    return W
