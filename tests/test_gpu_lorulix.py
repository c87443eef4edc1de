"""Lorulix on the GPU against the plain implementation in tests/lorulix_oracle.py: every mechanism alone, whole prompts,
token-by-token decoding, portions down to two tokens, unequal batches, reused blocks and state slots, far keys and the edges
of the distance buckets, the first tokens of a sequence, long decoding, odd sizes, hipGraph replays, swapping, and greedy
generation through the Engine and its scheduler. Configurations and weights are made here (small, random, seeded)."""
import asyncio
import json
import os

import pytest
import torch

import lorulix_oracle as O

pytestmark = pytest.mark.gpu

F32_TOL = 3e-5      # relative rms error of fp32 logits (true fp32 products, fp32 statistics)
BF16_TOL = 8e-2     # the same in bfloat16 (bf16 products and activations, fp32 stream, statistics and recurrences)


def write_model(path, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


def make_model(path, cfg, W, dtype="float32", num_blocks=48, max_seqs=4, cpu_blocks=0, graph=False):
    from swiftllm_amd import EngineConfig, build_model
    write_model(path, cfg, W)
    ecfg = EngineConfig(model_path=str(path), use_dummy=False, block_size=16, gpu_mem_utilization=0.9,
                        num_cpu_blocks=cpu_blocks, max_seqs_in_block_table=max_seqs,
                        max_blocks_per_seq=-(-cfg["max_positions"] // 16), max_batch_size=max_seqs,
                        max_tokens_in_batch=1024, dtype=dtype, use_hip_graph=graph)
    model = build_model(ecfg)
    model.load_weights()
    model.init_kvcache_and_swap(num_blocks)
    return model


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-9)).max())


def mostly_within(got, want, tol, share=0.75, median=True):
    """bfloat16 against the float64 oracle: rounding moves a router's close calls, and a token that goes to another expert
    differs by far more than rounding (and leaves a trace in the state of what follows). So the 16-bit runs are held to
    the tolerance at most positions and at the median; the fp32 runs of the same code are held to it everywhere."""
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-9)
    return (not median or float(e.median()) < tol / 2) and float((e < tol).double().mean()) >= share


def close(got, want, dtype, tol, share=0.75, median=True):
    return rel_err(got, want) < tol if dtype == "float32" else mostly_within(got, want, tol, share, median)


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def entry(seq, toks, start, want=None):
    from swiftllm_amd.worker.batch_plan import StepEntry
    return StepEntry(seq, toks, start, tuple(range(len(toks))) if want is None else tuple(want))


def run_in_portions(model, seq, toks, sizes):
    """Feed toks to sequence `seq` in portions of the given sizes (the last size repeats); -> logits of every position."""
    out, at, i = [], 0, 0
    while at < len(toks):
        n = min(sizes[min(i, len(sizes) - 1)], len(toks) - at)
        out.append(model.step([entry(seq, toks[at:at + n], at)]))
        at += n
        i += 1
    return torch.cat(out)


class Slots:
    """A StateSlotManager and the per-token arrays of hand-made steps, for the kernels that carry state."""

    def __init__(self, floats, num_slots=3):
        from swiftllm_amd.worker.state_slots import StateSlotManager
        self.mgr = StateSlotManager(num_slots)
        self.off = [self.mgr.add_region(f) for f in floats]
        self.mgr.allocate()
        self.mgr.pool.fill_(float("nan"))       # nothing may be read before it is written

    def ref(self, portions):
        """portions: [(seq id, start, count)] in batch order -> StateRef."""
        from swiftllm_amd.worker.kernels.rms_stream import StateRef
        codes = self.mgr.begin_step([p[0] for p in portions], [p[1] for p in portions])
        i32 = lambda xs: torch.tensor(xs, dtype=torch.int32, device="cuda")
        pos = [p[1] + j for p in portions for j in range(p[2])]
        start = [p[1] for p in portions for _ in range(p[2])]
        state = [int(c) for p, c in zip(portions, codes) for _ in range(p[2])]
        seq = [p[0] for p in portions for _ in range(p[2])]
        cnt = [p[2] for p in portions]
        row0 = [sum(cnt[:i]) for i in range(len(cnt))]
        return StateRef(self.mgr.pool, i32(pos), i32(start), i32(state), i32(seq), i32(row0), i32(cnt))


def interleave(lengths, cuts):
    """Steps for sequences of the given lengths cut at `cuts[i]` (portion sizes, the last repeats): a list of steps, each a
    list of (seq, start, count); sequences take turns and share steps."""
    at = [0] * len(lengths)
    k = [0] * len(lengths)
    steps = []
    while any(a < n for a, n in zip(at, lengths)):
        step = []
        for s, n in enumerate(lengths):
            if at[s] < n and (len(steps) + s) % 3 != 2:     # every sequence sits out some steps
                c = min(cuts[s][min(k[s], len(cuts[s]) - 1)], n - at[s])
                step.append((s, at[s], c))
                at[s] += c
                k[s] += 1
        if step:
            steps.append(step)
        else:
            steps.append([])
    return [s for s in steps if s]


# ---- mechanisms alone ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_stream_step(dtype):
    from swiftllm_amd.worker.kernels.rms_stream import gated_add_rmsnorm
    g = torch.Generator().manual_seed(0)
    n, w, eps = 37, 72, 1e-5
    x = torch.randn(n, w, generator=g) * 2 + 0.5
    m, m2 = (torch.randn(n, w, generator=g) * 3).to(dtype), (torch.randn(n, w, generator=g)).to(dtype)
    wide = torch.randn(n, w + 5, generator=g).to(dtype)         # the gate logits are a column slice of a wider matrix
    sgw = torch.randn(n, 3, generator=g).to(dtype)             # ... and so is the per-token gate of the second addend
    r, sg = wide[:, 2:2 + w], sgw[:, 1:2]
    rb, w1, w2 = torch.randn(w, generator=g), 1 + 0.3 * torch.randn(w, generator=g), 1 + 0.3 * torch.randn(w, generator=g)
    y = (m.double() + torch.sigmoid(sg.double()) * m2.double()) * torch.sigmoid(r.double() + rb.double())
    want_x = x.double() + O.unit_rms(y, eps) * w1.double()
    want_h = O.unit_rms(want_x, eps) * w2.double()
    xd = x.cuda()
    h = gated_add_rmsnorm(xd, m.cuda(), w1.cuda(), wide.cuda()[:, 2:2 + w], rb.cuda(), m2.cuda(), sgw.cuda()[:, 1:2],
                          pre=w2.cuda(), eps=eps)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert (xd.cpu().double() - want_x).abs().max() < 1e-4
    assert (h.cpu().double() - want_h).abs().max() < tol * 10
    rows = torch.tensor([5, 0, 36], dtype=torch.int32)
    got = gated_add_rmsnorm(xd, pre=w2.cuda(), eps=eps, out_dtype=dtype, row_idx=rows.cuda())
    assert (got.cpu().double() - want_h[rows.long()]).abs().max() < tol * 10
    # no gate, no second addend
    x2 = x.cuda()
    gated_add_rmsnorm(x2, m.cuda(), w1.cuda(), eps=eps)
    assert (x2.cpu().double() - (x.double() + O.unit_rms(m.double(), eps) * w1.double())).abs().max() < 1e-4


@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_causal_convolution_in_portions_and_reused_slots(taps):
    from swiftllm_amd.worker.kernels.rms_stream import causal_conv_state
    g = torch.Generator().manual_seed(taps)
    C = 40
    w = torch.randn(C, taps, generator=g)
    lengths = [23, 1, 9, 14]
    cuts = [[1, 2, 1, 7, 2, 3], [1], [2], [14]]
    hs = [torch.randn(n, C, generator=g) for n in lengths]
    want = [h.double() + O.causal_conv(h.double(), w.double()) for h in hs]
    slots = Slots([2 * (taps - 1) * C], num_slots=2)       # four sequences through two slots
    got = [[] for _ in lengths]
    live = []
    for pair in ((0, 1), (2, 3)):       # the second pair runs in the slots the first pair leaves
        for step in interleave([lengths[s] for s in pair], [cuts[s] for s in pair]):
            portions = [(pair[s], start, cnt) for s, start, cnt in step]
            st = slots.ref(portions)
            h = torch.cat([hs[s][start:start + cnt] for s, start, cnt in portions]).cuda()
            out = causal_conv_state(h, w.t().contiguous().cuda(), st, slots.off[0], add_input=True).cpu()
            at = 0
            for s, start, cnt in portions:
                got[s].append(out[at:at + cnt])
                at += cnt
        slots.mgr.release(list(pair))
    for s in range(len(lengths)):
        assert (torch.cat(got[s]).double() - want[s]).abs().max() < 1e-5


@pytest.mark.parametrize("H,G,d,e,conv,n", [(4, 2, 16, 16, 4, 70), (3, 1, 24, 40, 1, 33), (2, 2, 64, 64, 2, 40),
                                            (6, 2, 32, 48, 3, 300), (1, 1, 7, 5, 2, 20), (2, 1, 128, 128, 4, 24)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_delta_rule_in_portions(H, G, d, e, conv, n, dtype):
    """The recurrence, its convolutions and its output norm, cut into portions (single tokens and pairs among them), with a
    second sequence in the batch and the state slot of a finished sequence used again."""
    from swiftllm_amd.model_config import LorulixDeltaConfig
    from swiftllm_amd.worker.kernels.delta_rule import delta_rule_mixer
    g = torch.Generator().manual_seed(H * 100 + d)
    mx = {"heads": H, "kv_heads": G, "dim": d, "vdim": e, "conv": conv}
    mc = LorulixDeltaConfig(mx)
    eps = 1e-5
    W = {"q.conv": torch.randn(G * d, conv, generator=g) * 0.6, "k.conv": torch.randn(G * d, conv, generator=g) * 0.6,
         "v.conv": torch.randn(H * e, conv, generator=g) * 0.6, "A_log": torch.randn(H, generator=g) * 0.5,
         "dt_bias": torch.randn(H, generator=g) * 0.5, "norm": 1 + 0.2 * torch.randn(e, generator=g)}
    Wd = {k: v.double() for k, v in W.items()}
    conv_w = torch.cat((W["q.conv"], W["k.conv"], W["v.conv"])).t().contiguous().cuda()     # tap-major
    lengths = [n, 11]
    projs = [(torch.randn(m, mc.proj_size, generator=g) * 1.5).to(dtype) for m in lengths]
    want = []
    for p in projs:
        parts = torch.split(p.double(), [G * d, G * d, H * e, H * e, H, H], dim=1)
        want.append(O.delta_from_projections(*parts, Wd, "", mx, eps))
    slots = Slots([2 * (conv - 1) * mc.conv_channels, mc.state_elems], num_slots=2)
    # a sequence that ran before leaves its state in the slots
    junk = slots.ref([(7, 0, 5), (8, 0, 3)])
    delta_rule_mixer((torch.randn(8, mc.proj_size, generator=g)).to(dtype).cuda(), conv_w, W["A_log"].cuda(),
                     W["dt_bias"].cuda(), W["norm"].cuda(), junk, slots.off[0], slots.off[1], mc, eps)
    slots.mgr.release([7, 8])
    got = [[] for _ in lengths]
    for step in interleave(lengths, [[3, 1, 2, 1, 17, 2, 64], [2, 1]]):
        st = slots.ref(step)
        p = torch.cat([projs[s][start:start + cnt] for s, start, cnt in step]).cuda()
        out = delta_rule_mixer(p, conv_w, W["A_log"].cuda(), W["dt_bias"].cuda(), W["norm"].cuda(), st, slots.off[0],
                               slots.off[1], mc, eps).cpu()
        at = 0
        for s, start, cnt in step:
            got[s].append(out[at:at + cnt])
            at += cnt
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    for s in range(2):
        assert (torch.cat(got[s]).double() - want[s]).abs().max() < tol * max(1.0, float(want[s].abs().max()))


def test_distance_rows_match_the_bucket_function():
    from swiftllm_amd.model_config import distance_bias_rows
    for rows, far in ((12, 40), (32, 500), (7, 9), (2, 64), (16, 16.5)):
        assert distance_bias_rows(rows, far, 700) == [O.distance_bucket(n, rows, far) for n in range(700)]


def _attention_case(H, G, d, e, n, dtype, rel, temp, qkv, tiled, bias_max=40, chunks=(1000,)):
    """The store and attention kernels over a hand-made pool against the dense oracle; qkv [n, q | k | v] raw projections."""
    from swiftllm_amd.model_config import LorulixAttentionConfig
    from swiftllm_amd.worker.block_manager import BlockManager
    from swiftllm_amd.worker.kernels.window_attn import PoolSlice, qknorm_full_and_store_kv, window_attention
    mx = {"heads": H, "kv_heads": G, "dim": d, "vdim": e, "scale": 0.3, "bias_max": bias_max}
    if temp:
        mx["q_temp"] = {"coef": temp[0], "every": temp[1]}
    mc = LorulixAttentionConfig(mx)
    g = torch.Generator().manual_seed(n + H)
    qn, kn = 1 + 0.2 * torch.randn(H * d, generator=g), 1 + 0.2 * torch.randn(G * d, generator=g)
    eps = 1e-5
    qd = qkv.to(dtype).double()
    q = O.normed_queries(qd[:, :H * d], qn.double(), mx, eps)
    k = (O.unit_rms(qd[:, H * d:(H + G) * d], eps) * kn.double()).view(n, G, d)
    v = qd[:, (H + G) * d:].view(n, G, e)
    if dtype != torch.float32:      # what the pool and the query rows hold is rounded
        q, k = q.to(dtype).double(), k.to(dtype).double()
    want = O.attention_output(q, k, v, mx, rel.double() if rel is not None else None)
    blocks = -(-n // 16) + 3
    mgr = BlockManager("GPU", blocks + 5, 3, blocks, 16, "cuda")
    mgr.allocate_blocks_for_seqs([1], [37])         # another sequence owns the first blocks
    sl = PoolSlice(16 * 3, 16 * 3 + G * d * 16)     # (other layers' slices around it)
    # (finite garbage where nothing was stored: what a block that another sequence used before holds)
    pool = torch.full((blocks + 5, 16 * 3 + G * (d + e) * 16 + 32), 3e4, dtype=dtype, device="cuda")
    rel_dev = None
    if rel is not None:
        from swiftllm_amd.model_config import distance_bias_rows
        rel_dev = rel[torch.tensor(distance_bias_rows(rel.shape[0], bias_max, 512))].t().contiguous().float().cuda()
    out, at = [], 0
    for c in chunks * n:
        if at >= n:
            break
        c = min(c, n - at)
        mgr.allocate_blocks_for_seqs([2], [at + c])
        rows = qkv[at:at + c].to(dtype).cuda()
        pos = torch.arange(at, at + c, dtype=torch.int32, device="cuda")
        seq = torch.full((c,), 2, dtype=torch.int32, device="cuda")
        qknorm_full_and_store_kv(rows, qn.cuda(), kn.cuda(), pool, sl, mgr.block_table, seq, pos, mc, eps, True)
        tiles = None
        if tiled:
            r0 = torch.arange(0, c, 16, dtype=torch.int32)
            tiles = (r0.cuda(), torch.minimum(torch.full_like(r0, 16), c - r0).cuda())
        out.append(window_attention(rows, None, pool, sl, mgr.block_table, seq, pos, mc, tiles, 512, rel=rel_dev).cpu())
        at += c
    return torch.cat(out).double(), want


@pytest.mark.parametrize("H,G,d,e,n", [(4, 2, 16, 24, 150), (3, 1, 40, 8, 70), (2, 2, 8, 8, 1), (5, 5, 32, 16, 45)])
def test_attention_with_distance_bias(H, G, d, e, n):
    g = torch.Generator().manual_seed(n)
    qkv = torch.randn(n, H * d + G * (d + e), generator=g)
    rel = torch.randn(10, H, generator=g) * 1.5
    got, want = _attention_case(H, G, d, e, n, torch.float32, rel, (0.4, 8), qkv, False, chunks=(5, 1, 2, 30))
    assert (got - want).abs().max() < 2e-5
    got, want = _attention_case(H, G, d, e, n, torch.float32, None, None, qkv, False)
    assert (got - want).abs().max() < 2e-5


@pytest.mark.parametrize("H,G,d,e,n", [(4, 1, 64, 64, 150), (8, 2, 128, 64, 90), (3, 1, 64, 128, 37), (16, 4, 128, 128, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_matrix_core_attention_with_distance_bias(H, G, d, e, n, dtype):
    g = torch.Generator().manual_seed(n)
    qkv = torch.randn(n, H * d + G * (d + e), generator=g)
    rel = torch.randn(14, H, generator=g) * 1.5
    got, want = _attention_case(H, G, d, e, n, dtype, rel, (0.4, 8), qkv, True, chunks=(17, 1, 2, 40))
    assert (got - want).abs().max() < 2e-2
    plain, _ = _attention_case(H, G, d, e, n, dtype, rel, (0.4, 8), qkv, False, chunks=(17, 1, 2, 40))
    assert (got - plain).abs().max() < 2e-2


@pytest.mark.parametrize("tiled,dtype,d", [(False, torch.float32, 16), (True, torch.bfloat16, 64)])
def test_every_bucket_edge_shows_in_the_output(tiled, dtype, d):
    """One row of the bias table at a time is raised far above the scores: the output is then the mean of the values whose
    distance falls into that row, and a distance that is one off at a row's edge moves it."""
    H, G, e, n, rows, far = 2, 1, d, 130, 12, 100
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(n, H * d + G * (d + e), generator=g)
    qkv[:, :H * d] *= 0.05
    for row in range(rows):
        rel = torch.zeros(rows, H)
        rel[row] = 40.0
        got, want = _attention_case(H, G, d, e, n, dtype, rel, None, qkv, tiled, bias_max=far, chunks=(33, 1, 2))
        assert (got - want).abs().max() < (1e-4 if dtype == torch.float32 else 3e-2), f"row {row}"


@pytest.mark.parametrize("tiled,dtype,d", [(False, torch.float32, 24), (True, torch.bfloat16, 64)])
def test_a_far_key_among_hundreds_is_found(tiled, dtype, d):
    """The last queries point at one key hundreds of positions back (the same direction, so their score stands out); every
    other key is noise. In a prompt portion and as single decoded tokens."""
    H, G, e, n = 2, 1, d, 400
    g = torch.Generator().manual_seed(9)
    qkv = torch.randn(n, H * d + G * (d + e), generator=g)
    u = torch.randn(d, generator=g)
    qkv[13, H * d:(H + G) * d] = 4 * u
    qkv[-6:, :H * d] = 4 * u.repeat(H)
    rel = torch.randn(10, H, generator=g)
    got, want = _attention_case(H, G, d, e, n, dtype, rel, (0.5, 48), qkv, tiled, chunks=(397, 1))
    v13 = qkv[13, (H + G) * d:].to(dtype).double()
    assert (want[-1, :e] - v13).abs().max() < 0.2 * float(v13.abs().max())      # the oracle itself attends there
    assert (got - want).abs().max() < (2e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("n", [23, 300])       # per-assignment kernels / assignments sorted by expert + library products
@pytest.mark.parametrize("experts,top,shared", [(5, 2, 24), (70, 4, 0), (3, 3, 8), (4, 1, 0)])
def test_router_and_squared_relu_experts(experts, top, shared, n):
    from swiftllm_amd.worker.kernels.moe import moe_experts_relu2, moe_route_scores
    g = torch.Generator().manual_seed(experts)
    w, ff, scale = 48, 32, 1.7
    h = torch.randn(n, w, generator=g)
    W = {"router": torch.randn(experts, w, generator=g)}
    for x in range(experts):
        W[f"e{x}.up"] = torch.randn(ff, w, generator=g) * 0.3
        W[f"e{x}.down"] = torch.randn(w, ff, generator=g) * 0.3
    mlp = {"router": {"experts": experts, "top": top, "scale": scale}}
    up = torch.stack([W[f"e{x}.up"] for x in range(experts)]).cuda()
    down = torch.stack([W[f"e{x}.down"] for x in range(experts)]).cuda()
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 3e-2)):
        hd = h.to(dtype)
        Wd = {k: (v.double() if k == "router" else v.to(dtype).double()) for k, v in W.items()}
        want = O.moe_ff(hd.double(), Wd, "", mlp)
        s = torch.softmax(hd.double() @ Wd["router"].T, dim=-1)
        wts_want, idx_want = torch.topk(s, top, dim=-1)
        idx, wts = moe_route_scores(hd.cuda(), W["router"].cuda(), top, scale)
        assert torch.equal(idx.cpu().long(), idx_want)
        assert (wts.cpu().double() - scale * wts_want).abs().max() < 1e-5
        got = moe_experts_relu2(hd.cuda(), idx, wts, up.to(dtype), down.to(dtype))
        assert (got.cpu().double() - want).abs().max() < tol * max(1.0, float(want.abs().max()))


# ---- the whole model -------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def default_case():
    cfg = O.make_config()
    W = O.make_weights(cfg, seed=3)
    toks = tokens_for(cfg, 90, 1)
    logits, streams = O.forward(cfg, W, toks)
    return cfg, W, toks, logits, streams


@pytest.mark.parametrize("dtype,tol", [("float32", F32_TOL), ("bfloat16", BF16_TOL)])
def test_whole_prompt_logits_and_every_layer(tmp_path, default_case, dtype, tol):
    cfg, W, toks, want, streams = default_case
    model = make_model(tmp_path / "m", cfg, W, dtype)
    model.layer_tap = []
    got = model.step([entry(0, toks, 0)])
    assert len(model.layer_tap) == len(streams)
    for x, ref in zip(model.layer_tap, streams):
        if dtype == "float32":
            assert (x.cpu().double() - ref).abs().max() < 2e-4
        else:
            assert float((x.cpu().double() - ref).abs().median()) < 0.1
    assert close(got, want, dtype, tol)


@pytest.mark.parametrize("dtype,tol", [("float32", F32_TOL), ("bfloat16", BF16_TOL)])
def test_decoding_and_portions_match_the_whole_prompt(tmp_path, default_case, dtype, tol):
    cfg, W, toks, want, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, dtype)
    assert close(run_in_portions(model, 0, toks, [1]), want, dtype, tol)                    # token by token from the first
    assert close(run_in_portions(model, 1, toks, [2]), want, dtype, tol)                    # pairs
    assert close(run_in_portions(model, 2, toks, [3, 2, 16, 1, 31, 2, 17, 1]), want, dtype, tol)
    model.free_seqs_resources([0, 1, 2])
    assert close(run_in_portions(model, 0, toks, [58, 1]), want, dtype, tol)                # a prompt, then decoding


def test_decode_graph_replays_match_eager_steps(tmp_path, default_case):
    cfg, W, toks, want, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, "float32", graph=True)
    other = tokens_for(cfg, 70, 2)
    want_other = O.forward(cfg, W, other)[0]
    a = [model.step([entry(0, toks[:30], 0), entry(1, other[:11], 0)])]
    got0, got1 = [a[0][:30]], [a[0][30:]]
    for i in range(40):     # two sequences decode together: one captured graph, replayed with other positions and slots
        lg = model.step([entry(0, toks[30 + i:31 + i], 30 + i), entry(1, other[11 + i:12 + i], 11 + i)]).clone()
        got0.append(lg[:1])
        got1.append(lg[1:])
        torch.cuda.synchronize()
    assert model.graph_captures == 1
    assert rel_err(torch.cat(got0), want[:70]) < F32_TOL
    assert rel_err(torch.cat(got1), want_other[:51]) < F32_TOL


def test_unequal_batches_and_reused_blocks_and_slots(tmp_path, default_case):
    """Four live requests of unequal length, portions beside decoded tokens; finished requests give their blocks, block
    table rows and state slots to new ones. Every request's logits equal those of the request alone."""
    cfg, W, _, _, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, "float32", num_blocks=20, max_seqs=4)
    lens = [70, 5, 33, 1, 48, 17, 2]
    reqs = [tokens_for(cfg, n, 50 + i) for i, n in enumerate(lens)]
    wants = [O.forward(cfg, W, t)[0] for t in reqs]
    cuts = [[9, 1, 1, 30, 2], [2, 1], [33], [1], [16, 1], [3, 2], [1]]
    got = [[] for _ in reqs]
    at, k = [0] * len(reqs), [0] * len(reqs)
    waiting, live, rows = list(range(len(reqs))), {}, [3, 2, 1, 0]
    steps = 0
    while waiting or live:
        while waiting and rows:
            live[waiting.pop(0)] = rows.pop()
        batch, ended = [], []
        for r, row in live.items():
            if (steps + r) % 4 == 3 and len(live) > 1:
                continue        # a request that sits a step out
            c = min(cuts[r][min(k[r], len(cuts[r]) - 1)], lens[r] - at[r])
            batch.append((r, entry(row, reqs[r][at[r]:at[r] + c], at[r])))
            at[r] += c
            k[r] += 1
        if batch:
            lg = model.step([e for _, e in batch])
            o = 0
            for r, e in batch:
                got[r].append(lg[o:o + len(e.tokens)])
                o += len(e.tokens)
                if at[r] == lens[r]:
                    ended.append(r)
        for r in ended:
            model.free_seqs_resources([live[r]])
            rows.append(live.pop(r))
        steps += 1
    assert model.gpu_block_manager.num_free_blocks == 20 and model.state.num_free_slots == 4
    for r in range(len(reqs)):
        assert rel_err(torch.cat(got[r]), wants[r]) < F32_TOL, f"request {r}"


def varied_config():
    """Sizes that a symmetric configuration would hide: dim != vdim, heads not a power of two, one kv head, heads = kv heads,
    a layer without feed-forward, top = 1 and top = experts, experts without a shared one, a delta layer first, convolutions
    of one tap, two layers that borrow the same keys, no distance bias, no temperature, a temperature that grows every token."""
    layers = [
        O.delta_layer(heads=3, kv_heads=1, dim=24, vdim=8, conv=1, mlp=O.moe_mlp(40, 6, 1)),
        O.attention_layer(heads=6, kv_heads=3, dim=16, vdim=24, bias_max=90, temp=(0.7, 1), mlp=None),
        O.attention_layer(heads=3, kv_heads=1, dim=24, vdim=8, bias_max=None, temp=None, mlp=O.dense_mlp(72, limit=0.6)),
        O.delta_layer(heads=2, kv_heads=2, dim=8, vdim=40, conv=5, mlp=O.moe_mlp(24, 3, 3, scale=0.5, shared=16)),
        O.attention_layer(heads=6, kv_heads=3, dim=16, vdim=24, bias_max=17, temp=(0.2, 5), kv_from=1, mlp=O.dense_mlp(56)),
        O.attention_layer(heads=6, kv_heads=3, dim=16, vdim=24, bias_max=None, kv_from=1, mlp=None),
    ]
    return O.make_config(width=40, vocab=70, layers=layers, taps=2, max_positions=160)


@pytest.mark.parametrize("dtype,tol", [("float32", F32_TOL), ("bfloat16", BF16_TOL)])
@pytest.mark.parametrize("taps", [2, 1, 4])
def test_other_sizes(tmp_path, dtype, tol, taps):
    cfg = varied_config()
    cfg["canon"]["taps"] = taps
    W = O.make_weights(cfg, seed=11, bias_rows=9)
    toks = tokens_for(cfg, 75, 4)
    want = O.forward(cfg, W, toks)[0]
    model = make_model(tmp_path / "m", cfg, W, dtype)
    # (bfloat16: top = 1 in the first layer and attention layers after it — one moved choice early in a short sequence
    # colours every later position, so only the positions ahead of it are held to the oracle; float32 holds them all)
    whole, cut = model.step([entry(0, toks, 0)]), run_in_portions(model, 1, toks, [2, 1, 20, 3, 1])
    assert close(whole, want, dtype, tol, share=0.05, median=False)
    assert close(cut, want, dtype, tol, share=0.05, median=False)
    assert rel_err(whole[:3], want[:3]) < tol and rel_err(cut[:3], want[:3]) < tol


def random_config(rng):
    """A configuration drawn at random: layer order, head counts and sizes (also ones no kernel is specialised for), taps,
    experts, which layers borrow keys, which constants are present."""
    layers, own = [], []
    for i in range(rng.randint(3, 5)):
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            mlp = None
        elif kind == "dense":
            mlp = O.dense_mlp(rng.choice([64, 100, 176]), limit=rng.choice([0.8, 1.7, 7.0]))
        else:
            experts = rng.choice([2, 4, 8, 16])
            mlp = O.moe_mlp(rng.choice([16, 48, 80]), experts, rng.randint(1, min(experts, 4)), scale=rng.choice([1.0, 2.0, 0.5]),
                            shared=rng.choice([None, 32, 72]))
        r = rng.random()
        if r < 0.4:
            kv = rng.choice([1, 2, 3])
            layers.append(O.delta_layer(heads=kv * rng.choice([1, 2, 3]), kv_heads=kv, dim=rng.choice([16, 24, 32, 64, 128]),
                                        vdim=rng.choice([16, 40, 64, 128]), conv=rng.choice([1, 2, 3, 4]), mlp=mlp))
        elif r < 0.75 or not own:
            kv = rng.choice([1, 2, 4])
            layers.append(O.attention_layer(heads=kv * rng.choice([1, 2, 3]), kv_heads=kv, dim=rng.choice([16, 32, 48, 64, 128]),
                                            vdim=rng.choice([16, 32, 64, 128]), scale=rng.choice([0.11, 0.3, 0.08]),
                                            bias_max=rng.choice([None, 30, 200, 1000]),
                                            temp=rng.choice([None, (0.5, 48), (0.3, 7), (1.0, 1)]), mlp=mlp))
            own.append(i)
        else:
            j = rng.choice(own)
            src = layers[j]["mixer"]
            layers.append(O.attention_layer(heads=src["heads"], kv_heads=src["kv_heads"], dim=src["dim"], vdim=src["vdim"],
                                            scale=rng.choice([0.15, 0.2]), bias_max=rng.choice([None, 64, 500]),
                                            temp=rng.choice([None, (0.5, 16)]), kv_from=j, mlp=mlp))
    return O.make_config(width=rng.choice([64, 96, 160]), vocab=rng.choice([100, 300, 577]), layers=layers,
                         taps=rng.choice([1, 2, 3, 4]), max_positions=256, eps=rng.choice([1e-5, 1e-6]))


@pytest.mark.parametrize("seed", [1, 4, 8, 9])
def test_random_configurations_in_a_mixed_batch(tmp_path, seed):
    """Three requests of a randomly drawn model in random portions (single tokens, pairs, page-sized and longer ones) that
    share steps and sit steps out; every request equals the oracle on the request alone, in float32 at every position. A
    random model has positions where rounding alone is amplified (a plain float32 evaluation of the oracle differs from the
    float64 one by up to 2e-5 at single positions of these models, 1e-6 at the median), hence a median and a maximum."""
    import random
    rng = random.Random(seed)
    cfg = random_config(rng)
    W = O.make_weights(cfg, seed=seed, bias_rows=rng.choice([8, 13, 32]))
    reqs = [tokens_for(cfg, n, seed * 10 + i) for i, n in enumerate((120, 37, 64))]
    wants = [O.forward(cfg, W, t)[0] for t in reqs]
    model = make_model(tmp_path / "m", cfg, W, "float32", num_blocks=20, max_seqs=3)
    at, got = [0, 0, 0], [[], [], []]
    while any(a < len(r) for a, r in zip(at, reqs)):
        batch = []
        for i in range(3):
            if at[i] < len(reqs[i]) and rng.random() < 0.8:
                c = min(rng.choice([1, 1, 2, 3, 16, 17, 40]), len(reqs[i]) - at[i])
                batch.append((i, entry(i, reqs[i][at[i]:at[i] + c], at[i])))
                at[i] += c
        if batch:
            lg = model.step([e for _, e in batch])
            o = 0
            for i, e in batch:
                got[i].append(lg[o:o + len(e.tokens)])
                o += len(e.tokens)
    for i in range(3):
        g, w = torch.cat(got[i]).double().cpu(), wants[i]
        d = g - w
        d = d - d.mean(-1, keepdim=True)
        e = d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt()
        assert float(e.median()) < 5e-6 and float(e.max()) < 2e-4, f"request {i} of {cfg['layers']}"


def test_matrix_core_paths_in_the_model(tmp_path):
    """bfloat16 with heads of 64 / 128: the tiled attention with its bias, the expert-stationary kernels, the packed decode
    projections — a prompt in portions and decoded tokens against the oracle on the same (bf16-representable) weights."""
    layers = [O.attention_layer(heads=8, kv_heads=2, dim=64, vdim=128, bias_max=120, mlp=O.moe_mlp(64, 8, 2, shared=64)),
              O.delta_layer(heads=4, kv_heads=2, dim=64, vdim=64, conv=4, mlp=O.dense_mlp(256)),
              O.attention_layer(heads=8, kv_heads=2, dim=64, vdim=128, bias_max=120, kv_from=0, mlp=O.moe_mlp(64, 8, 2))]
    cfg = O.make_config(width=128, vocab=160, layers=layers, max_positions=256)
    W = O.make_weights(cfg, seed=5, bias_rows=16)
    toks = tokens_for(cfg, 140, 6)
    want = O.forward(cfg, W, toks)[0]
    model = make_model(tmp_path / "m", cfg, W, "bfloat16")
    assert mostly_within(model.step([entry(0, toks, 0)]), want, BF16_TOL)
    assert mostly_within(run_in_portions(model, 1, toks, [33, 2, 64, 1]), want, BF16_TOL)


def test_first_tokens_of_a_sequence(tmp_path, default_case):
    """Sequences shorter than the convolutions, alone and decoded, in slots that longer sequences used before."""
    cfg, W, toks, want, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, "float32", max_seqs=2)
    model.step([entry(0, toks, 0, want=[]), entry(1, toks[::-1], 0, want=[])])
    model.free_seqs_resources([0, 1])
    for n in (1, 2, 3, 4):
        assert rel_err(model.step([entry(0, toks[:n], 0)]), want[:n]) < F32_TOL
        assert rel_err(run_in_portions(model, 1, toks[:n], [1]), want[:n]) < F32_TOL
        model.free_seqs_resources([0, 1])


def test_long_decoding(tmp_path):
    cfg = O.make_config(max_positions=400)
    W = O.make_weights(cfg, seed=8)
    toks = tokens_for(cfg, 330, 3)
    want = O.forward(cfg, W, toks)[0]
    model = make_model(tmp_path / "m", cfg, W, "float32", num_blocks=24)
    assert rel_err(run_in_portions(model, 0, toks, [10, 1]), want) < F32_TOL


def test_swap_out_and_in_keeps_the_sequence(tmp_path, default_case):
    cfg, W, toks, want, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, "float32", num_blocks=12, cpu_blocks=8, max_seqs=2)
    first = model.step([entry(0, toks[:40], 0)])
    model.swap_out_seqs([0])
    assert model.gpu_block_manager.num_free_blocks == 12 and model.state.num_free_slots == 2
    model.step([entry(1, tokens_for(cfg, 100, 1), 0, want=[])])      # overwrites the freed blocks and the freed slot
    model.free_seqs_resources([1])
    model.step([entry(1, tokens_for(cfg, 30, 2), 0, want=[])])
    model.swap_in_seqs([0])
    rest = model.step([entry(0, toks[40:], 40)])
    assert rel_err(torch.cat((first, rest)), want) < F32_TOL


def test_greedy_generation_through_the_engine(tmp_path, default_case):
    """The framework's own entry point: Engine + scheduler + worker protocol, whole prompts then decoding, requests of
    unequal length finishing at different times."""
    from swiftllm_amd import EngineConfig
    from swiftllm_amd.server import Engine, RawRequest
    cfg, W, _, _, _ = default_case
    path = write_model(tmp_path / "m", cfg, W)
    ecfg = EngineConfig(model_path=path, use_dummy=False, block_size=16, gpu_mem_utilization=0.12, num_cpu_blocks=8,
                        max_seqs_in_block_table=4, max_blocks_per_seq=16, max_batch_size=4, max_tokens_in_batch=256,
                        dtype="float32", use_hip_graph=True)
    prompts = [tokens_for(cfg, n, 20 + n) for n in (5, 33, 18)]
    outs = (6, 12, 9)

    def oracle(prompt, n):
        seq = list(prompt)
        for _ in range(n):
            lg = O.forward(cfg, W, seq)[0][-1]
            top2 = torch.topk(lg, 2).values
            assert float(top2[0] - top2[1]) > 1e-4, "the test's weights make a close call"
            seq.append(int(torch.argmax(lg)))
        return seq[len(prompt):]

    async def run():
        engine = Engine(ecfg)
        await engine.initialize()
        assert type(engine.model).__name__ == "LorulixModel"
        loops = asyncio.ensure_future(engine.start_all_event_loops())
        res = await asyncio.gather(*[engine.add_request_and_wait(RawRequest("", n, p)) for p, n in zip(prompts, outs)])
        loops.cancel()
        try:
            await loops
        except (asyncio.CancelledError, Exception):
            pass
        return [r[1] for r in res]

    got = asyncio.run(run())
    import gc
    gc.collect()                    # (the engine's pool goes back before the next test sizes its own)
    torch.cuda.empty_cache()
    for g, p, n in zip(got, prompts, outs):
        assert g == oracle(p, n)
