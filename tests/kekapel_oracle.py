"""A plain, slow Kekapel for the tests: one function per mechanism, whole sequences, float64, dense masks.

Nothing here is shared with swiftllm_amd: the product computes the same design with paged caches and HIP kernels, this
file with full [tokens, tokens] score matrices and Python loops. `weights` is a dict name -> tensor with the checkpoint's
tensor names, `cfg` the parsed config.json.
"""
import math

import torch

F64 = torch.float64


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def window_mask(n, size):
    """[n, n] bool: query i sees key j iff 0 <= i - j < size (size None: every earlier key)."""
    i = torch.arange(n).unsqueeze(1)
    j = torch.arange(n).unsqueeze(0)
    d = i - j
    m = d >= 0
    if size is not None:
        m &= d < size
    return m


def head_scores(q, k, mx, eps, qn, kn):
    """q [n, H, d], k [n, G, d] -> capped scores [H, n, n] before the heads are mixed."""
    H, G = mx["heads"], mx["kv_heads"]
    q = unit_rms(q, eps) * qn
    k = unit_rms(k, eps) * kn
    k = k.repeat_interleave(H // G, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, k) * mx["scale"]
    cap = mx.get("softcap")
    if cap:
        s = cap * torch.tanh(s / cap)
    return s


def mix_heads(s, talk):
    """s [H, n, n], talk [H, H]: out[h] = sum_g talk[h, g] s[g]."""
    return torch.einsum("hg,gij->hij", talk, s)


def attention_mixer(h, W, pre, mx, eps):
    n = h.shape[0]
    H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = (h @ W[pre + "q"].T).view(n, H, d)
    k = (h @ W[pre + "k"].T).view(n, G, d)
    v = (h @ W[pre + "v"].T).view(n, G, dv).repeat_interleave(H // G, dim=1)
    s = head_scores(q, k, mx, eps, W[pre + "q.norm"], W[pre + "k.norm"])
    s = mix_heads(s, W[pre + "talk"])
    size = (mx.get("mask") or {}).get("size")
    s = s.masked_fill(~window_mask(n, size), float("-inf"))
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("hij,jhd->ihd", p, v).reshape(n, H * dv)
    return o @ W[pre + "o"].T


def polynorm(z, act, eps):
    a, b, c, e = [float(x) for x in act]
    return a * unit_rms(z, eps) + b * unit_rms(z ** 2, eps) + c * unit_rms(z ** 3, eps) + e


def dense_ff(h, W, pre, eps):
    return polynorm(h @ W[pre + "up"].T, W[pre + "act"], eps) @ W[pre + "down"].T


def route(h, W, pre, top):
    """-> (chosen experts [n, top], their weights [n, top])."""
    z = h @ W[pre + "router"].T + W[pre + "router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def expert_ff(h, W, pre, limit):
    g = torch.clamp(h @ W[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ W[pre + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[pre + "down"].T


def moe_ff(h, W, pre, mlp):
    idx, wts = route(h, W, pre, mlp["router"]["top"])
    out = torch.zeros(h.shape[0], W[pre + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            e = int(idx[t, j])
            out[t] += wts[t, j] * expert_ff(h[t:t + 1], W, f"{pre}e{e}.", mlp["expert"]["limit"])[0]
    return out


def layer_runs(cfg):
    """Order in which layers run: [(layer index, pass number or None, first of its pass)]."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    out = [(i, None, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        for i in range(loop["start"], loop["stop"]):
            out.append((i, t, i == loop["start"]))
    out += [(i, None, False) for i in range(loop["stop"], n)]
    return out


def forward(cfg, weights, tokens, trace=None):
    """tokens: list of ids of ONE sequence from position 0 -> logits [n, vocab] float64. `trace`: a list that receives
    the residual stream after every layer run."""
    W = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    ids = torch.tensor(tokens, dtype=torch.long)
    n = ids.numel()
    x = W["embed"][ids] * cfg["embedding"]["scale"] + W["pos"][:n]
    x0 = x.clone()
    for i, t, first in layer_runs(cfg):
        if first:
            if t > 0:
                x = x + x0
            x = x + W["loop.step"][t]
        L, p = cfg["layers"][i], f"l{i}."
        assert L["type"] == "attention"
        y = attention_mixer(layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps), W, p + "mix.", L["mixer"], eps)
        x = x + m * layer_norm(y, W[p + "norm1b"], W[p + "norm1b.b"], eps)
        if L.get("mlp"):
            h = layer_norm(x, W[p + "norm2"], W[p + "norm2.b"], eps)
            y = dense_ff(h, W, p + "mlp.", eps) if L["mlp"]["kind"] == "dense" else moe_ff(h, W, p + "mlp.", L["mlp"])
            x = x + m * layer_norm(y, W[p + "norm2b"], W[p + "norm2b.b"], eps)
        if trace is not None:
            trace.append(x.clone())
    x = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    return x @ W["head"].T


def random_weights(cfg, seed=0, dtype=torch.bfloat16, spread=1.0):
    """Checkpoint tensors for a configuration (name -> tensor), values already rounded to `dtype`."""
    g = torch.Generator().manual_seed(seed)
    wd, out = cfg["width"], {}

    def mat(o, i, s=1.0):
        return (torch.randn(o, i, generator=g) * (s * spread / math.sqrt(i))).to(dtype)

    def vec(n, mean=0.0, s=0.1):
        return (mean + torch.randn(n, generator=g) * s).to(dtype)

    out["embed"] = (torch.randn(cfg["vocab"], wd, generator=g) * 0.1).to(dtype)
    out["pos"] = (torch.randn(cfg["max_positions"], wd, generator=g) * 0.3).to(dtype)
    if cfg.get("loop"):
        out["loop.step"] = (torch.randn(cfg["loop"]["times"], wd, generator=g) * 0.3).to(dtype)
    for i, L in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", L["mixer"]
        for nm in ("norm1", "norm2", "norm1b", "norm2b"):
            if nm.startswith("norm2") and not L.get("mlp"):
                continue
            out[p + nm] = vec(wd, 1.0)
            out[p + nm + ".b"] = vec(wd, 0.0)
        H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        out[p + "mix.q"] = mat(H * d, wd)
        out[p + "mix.k"] = mat(G * d, wd)
        out[p + "mix.v"] = mat(G * dv, wd)
        out[p + "mix.q.norm"] = vec(d, 1.0, 0.3)
        out[p + "mix.k.norm"] = vec(d, 1.0, 0.3)
        out[p + "mix.talk"] = (torch.eye(H) + torch.randn(H, H, generator=g) * 0.3).to(dtype)
        out[p + "mix.o"] = mat(wd, H * dv)
        mlp = L.get("mlp")
        if not mlp:
            continue
        if mlp["kind"] == "dense":
            out[p + "mlp.up"] = mat(mlp["ff"], wd)
            out[p + "mlp.down"] = mat(wd, mlp["ff"])
            out[p + "mlp.act"] = torch.tensor([0.7, 0.4, -0.3, 0.05]).add(torch.randn(4, generator=g) * 0.1).to(dtype)
        else:
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                out[f"{p}mlp.e{e}.gate"] = mat(ff, wd, 2.0)
                out[f"{p}mlp.e{e}.up"] = mat(ff, wd, 2.0)
                out[f"{p}mlp.e{e}.down"] = mat(wd, ff)
            out[p + "mlp.router"] = mat(mlp["router"]["experts"], wd, 3.0)
            out[p + "mlp.router.b"] = vec(mlp["router"]["experts"], 0.0, 0.5)
    out["final.norm"] = vec(wd, 1.0)
    out["final.norm.b"] = vec(wd, 0.0)
    out["head"] = mat(cfg["vocab"], wd)
    return out


def make_config(width=64, vocab=96, layers=None, loop=None, max_positions=256, eps=1e-5, residual_mult=0.5,
                embedding_scale=3.0):
    if layers is None:
        layers = [attention_layer(mlp=dense_mlp(96)), attention_layer(mlp=moe_mlp(48, 5, 2))]
    cfg = {"architecture": "Kekapel", "embedding": {"scale": embedding_scale}, "layers": layers,
           "max_positions": max_positions, "norm": {"eps": eps}, "residual_mult": residual_mult, "vocab": vocab,
           "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, window=9, scale=0.3, softcap=8.0, mlp=None):
    return {"type": "attention", "mlp": mlp,
            "mixer": {"dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"size": window}, "scale": scale,
                      "softcap": softcap, "vdim": vdim}}


def dense_mlp(ff):
    return {"kind": "dense", "ff": ff}


def moe_mlp(ff, experts, top, limit=1.5):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
