"""Kekapel on the GPU against the plain implementation in tests/kekapel_oracle.py: every mechanism alone, whole prompts,
token-by-token decoding, portions, unequal batches, reused blocks and rows, window edges, odd sizes, and greedy generation
through the Engine and its scheduler. Configurations and weights are made here (small, random, seeded)."""
import asyncio
import json
import os

import pytest
import torch

import kekapel_oracle as O

pytestmark = pytest.mark.gpu

F32_TOL = 3e-5      # relative rms error of fp32 logits (true fp32 products, fp32 statistics)
BF16_TOL = 4e-2     # the same in bfloat16 (bf16 products and activations, fp32 stream and statistics)


def write_model(path, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


def make_model(path, cfg, W, dtype="float32", num_blocks=48, max_seqs=4, cpu_blocks=0):
    from swiftllm_amd import EngineConfig, build_model
    write_model(path, cfg, W)
    ecfg = EngineConfig(model_path=str(path), use_dummy=False, block_size=16, gpu_mem_utilization=0.9,
                        num_cpu_blocks=cpu_blocks, max_seqs_in_block_table=max_seqs,
                        max_blocks_per_seq=-(-cfg["max_positions"] // 16), max_batch_size=max_seqs,
                        max_tokens_in_batch=1024, dtype=dtype, use_hip_graph=False)
    model = build_model(ecfg)
    model.load_weights()
    model.init_kvcache_and_swap(num_blocks)
    return model


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-9)).max())


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def entry(seq, toks, start, want=None):
    from swiftllm_amd.worker.batch_plan import StepEntry
    return StepEntry(seq, toks, start, tuple(range(len(toks))) if want is None else tuple(want))


def varied_config():
    """Sizes that a symmetric configuration would hide: dim != vdim, heads not a power of two, one kv head, window 1, a
    layer without feed-forward, top = 1 and top = experts, a loop that starts at layer 0."""
    layers = [
        O.attention_layer(heads=6, kv_heads=3, dim=16, vdim=24, window=7, mlp=O.moe_mlp(40, 6, 1)),
        O.attention_layer(heads=3, kv_heads=1, dim=24, vdim=8, window=1, mlp=None),
        O.attention_layer(heads=4, kv_heads=4, dim=8, vdim=16, window=300, softcap=None, mlp=O.dense_mlp(72)),
        O.attention_layer(heads=2, kv_heads=1, dim=40, vdim=40, window=33, scale=0.2, mlp=O.moe_mlp(24, 3, 3, limit=0.7)),
    ]
    return O.make_config(width=48, vocab=80, layers=layers, loop=(0, 2, 2), max_positions=160)


# ---- mechanisms alone ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_layernorm_and_fused_step(dtype):
    from swiftllm_amd.worker.kernels.layernorm import add_layernorm, layernorm
    g = torch.Generator().manual_seed(0)
    n, w, eps = 37, 72, 1e-5
    x = torch.randn(n, w, generator=g) * 2 + 0.5
    y = (torch.randn(n, w, generator=g) * 3).to(dtype)
    x0, step = torch.randn(n, w, generator=g), torch.randn(w, generator=g)
    w1, b1, w2, b2 = (torch.randn(w, generator=g) for _ in range(4))
    want_x = x.double() + 0.3 * O.layer_norm(y.double(), w1.double(), b1.double(), eps) + x0.double() + step.double()
    want_h = O.layer_norm(want_x, w2.double(), b2.double(), eps)
    xd = x.cuda()
    h = add_layernorm(xd, y.cuda(), 0.3, (w1.cuda(), b1.cuda()), x0.cuda(), step.cuda(), (w2.cuda(), b2.cuda()), eps)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert (xd.cpu().double() - want_x).abs().max() < 1e-4
    assert (h.cpu().double() - want_h).abs().max() < tol * 10
    rows = torch.tensor([5, 0, 36], dtype=torch.int32)
    got = layernorm(xd, w2.cuda(), b2.cuda(), eps, dtype, rows.cuda())
    assert (got.cpu().double() - want_h[rows.long()]).abs().max() < tol * 10


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_polynorm(dtype):
    from swiftllm_amd.worker.kernels.polynorm import polynorm
    z = (torch.randn(19, 100, generator=torch.Generator().manual_seed(1)) * 1.7).to(dtype)
    act = [0.7, -0.4, 0.25, 0.1]
    want = O.polynorm(z.double(), act, 1e-6)
    got = polynorm(z.cuda(), act, 1e-6).cpu().double()
    assert (got - want).abs().max() < (1e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("n", [23, 300])       # per-assignment kernels / assignments sorted by expert + library products
@pytest.mark.parametrize("experts,top", [(5, 2), (70, 4), (3, 3), (4, 1)])
def test_moe_router_and_experts(experts, top, n):
    from swiftllm_amd.worker.kernels import moe
    from swiftllm_amd.worker.kernels.moe import moe_experts, moe_route
    g = torch.Generator().manual_seed(experts)
    w, ff, limit = 40, 24, 0.9
    assert (300 * 2 >= moe.GROUPED_MIN_ROWS_PER_EXPERT * 5) and (23 * 2 < moe.GROUPED_MIN_ROWS_PER_EXPERT * 5)   # both paths run
    h = torch.randn(n, w, generator=g)
    W = {"router": torch.randn(experts, w, generator=g), "router.b": torch.randn(experts, generator=g)}
    for e in range(experts):
        W[f"e{e}.gate"] = torch.randn(ff, w, generator=g) * 0.3
        W[f"e{e}.up"] = torch.randn(ff, w, generator=g) * 0.3
        W[f"e{e}.down"] = torch.randn(w, ff, generator=g) * 0.3
    Wd = {k: v.double() for k, v in W.items()}
    idx_want, wts_want = O.route(h.double(), Wd, "", top)
    idx, wts = moe_route(h.cuda(), W["router"].cuda(), W["router.b"].cuda(), top)
    assert torch.equal(idx.cpu().long(), idx_want)
    assert (wts.cpu().double() - wts_want).abs().max() < 1e-6
    mlp = {"router": {"top": top}, "expert": {"limit": limit}}
    want = O.moe_ff(h.double(), Wd, "", mlp)
    gate_up = torch.stack([torch.cat((W[f"e{e}.gate"], W[f"e{e}.up"])) for e in range(experts)]).cuda()
    down = torch.stack([W[f"e{e}.down"] for e in range(experts)]).cuda()
    got = moe_experts(h.cuda(), idx, wts, gate_up, down, limit)
    assert (got.cpu().double() - want).abs().max() < 2e-5
    # 16-bit: decode-sized steps take the expert-stationary kernels (weights in registers, assignments grouped by expert in
    # the kernel), large ones the sorted library products; same routing, results within 16-bit rounding of the oracle on
    # the rounded inputs
    hb = h.to(torch.bfloat16)
    Wb = {k: v.to(torch.bfloat16).double() for k, v in W.items()}
    Wb["router"], Wb["router.b"] = Wd["router"], Wd["router.b"]
    want_b = O.moe_ff(hb.double(), Wb, "", mlp)
    idx_b, wts_b = moe_route(hb.cuda(), W["router"].cuda(), W["router.b"].cuda(), top)
    assert torch.equal(idx_b.cpu().long(), O.route(hb.double(), Wb, "", top)[0])
    got_b = moe_experts(hb.cuda(), idx_b, wts_b, gate_up.to(torch.bfloat16), down.to(torch.bfloat16), limit)
    assert (got_b.cpu().double() - want_b).abs().max() < 3e-2 * max(1.0, float(want_b.abs().max()))


def _attention_case(heads, kv_heads, dim, vdim, window, n, softcap, seed, standout=None, dtype=torch.float32, tiled=False,
                    cuts=None):
    """One mixer over a sequence of n tokens held in scattered blocks, fed as two portions and one decoded token, against
    the dense-mask oracle. standout = (query, key): that pair's score is made to dominate its row."""
    from swiftllm_amd.model_config import KekapelMixerConfig
    from swiftllm_amd.worker.kernels import window_attn
    from swiftllm_amd.worker.kernels.window_attn import PoolSlice, qknorm_and_store_kv, window_attention
    g = torch.Generator().manual_seed(seed)
    mxd = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 0.35, "softcap": softcap,
           "mask": {"size": window}}
    mixer = KekapelMixerConfig(mxd)
    q = torch.randn(n, heads, dim, generator=g)
    k = torch.randn(n, kv_heads, dim, generator=g)
    v = torch.randn(n, kv_heads, vdim, generator=g)
    if standout is not None:
        qi, kj = standout
        k[kj] = torch.randn(kv_heads, dim, generator=g) * 6
        q[qi] = k[kj].repeat_interleave(heads // kv_heads, dim=0) * 1.5
    qn, kn = 1 + 0.3 * torch.randn(dim, generator=g), 1 + 0.3 * torch.randn(dim, generator=g)
    talk = torch.eye(heads) + 0.4 * torch.randn(heads, heads, generator=g)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    eps = 1e-5
    s = O.head_scores(q.double(), k.double(), mxd, eps, qn.double(), kn.double())
    s = O.mix_heads(s, talk.double()).masked_fill(~O.window_mask(n, window), float("-inf"))
    p = torch.softmax(s, -1)
    want = torch.einsum("hij,jhd->ihd", p, v.double().repeat_interleave(heads // kv_heads, dim=1)).reshape(n, -1)

    blocks = -(-n // 16)
    num_blocks = blocks + 5
    perm = torch.randperm(num_blocks, generator=g)[:blocks].to(torch.int32)
    table = torch.full((3, blocks + 2), -1, dtype=torch.int32)
    table[1, :blocks] = perm
    pad = 24    # the run's slice sits in the middle of a wider block (other runs on both sides)
    block_elems = pad + 16 * kv_heads * (dim + vdim) + 8
    pool = torch.zeros(num_blocks, block_elems, dtype=dtype).cuda()
    sl = PoolSlice(pad, pad + 16 * kv_heads * dim)
    qkv = torch.cat((q.reshape(n, -1), k.reshape(n, -1), v.reshape(n, -1)), dim=1).cuda()
    seq = torch.full((n,), 1, dtype=torch.int32).cuda()
    pos = torch.arange(n, dtype=torch.int32).cuda()
    table = table.cuda()
    out = []
    if cuts is None:
        cuts = [0, max(1, n // 3), n - 1, n] if n > 2 else [0, n]
    saved = window_attn.TILES_MIN_TOKENS
    window_attn.TILES_MIN_TOKENS = 1 if tiled else saved
    try:
        for a, b in zip(cuts[:-1], cuts[1:]):
            if a == b:
                continue
            part = qkv[a:b].contiguous()
            qknorm_and_store_kv(part, qn.cuda(), kn.cuda(), pool, sl, table, seq[a:b], pos[a:b], mixer, eps)
            tiles = None
            if tiled:
                assert window_attn.tiles_supported(mixer, dtype)
                starts = torch.arange(0, b - a, 16, dtype=torch.int32)
                tiles = (starts.cuda(), torch.clamp(b - a - starts, max=16).to(torch.int32).cuda())
            out.append(window_attention(part, talk.cuda(), pool, sl, table, seq[a:b], pos[a:b], mixer, tiles))
    finally:
        window_attn.TILES_MIN_TOKENS = saved
    got = torch.cat(out).cpu().double()
    return got, want


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,window,n", [
    (4, 2, 16, 16, 9, 50), (6, 2, 64, 48, 36, 150), (3, 1, 24, 8, 1, 20), (5, 5, 8, 40, 200, 70), (2, 1, 72, 16, 64, 130),
    (8, 2, 32, 32, 16, 33), (1, 1, 16, 16, 5, 18)])
def test_window_attention_against_dense_mask(heads, kv_heads, dim, vdim, window, n):
    got, want = _attention_case(heads, kv_heads, dim, vdim, window, n, 6.0, seed=n)
    assert (got - want).abs().max() < 2e-5
    got, want = _attention_case(heads, kv_heads, dim, vdim, window, n, None, seed=n + 1, dtype=torch.bfloat16)
    assert (got - want).abs().max() < 8e-2     # (q and k are rounded to bfloat16 after their norms; scores reach +-20 here)


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,window,n", [
    (6, 2, 64, 64, 36, 150), (8, 2, 128, 128, 9, 70), (16, 4, 128, 64, 64, 131), (32, 8, 64, 64, 33, 90),
    (5, 5, 64, 128, 200, 100), (1, 1, 64, 64, 16, 49), (3, 1, 128, 128, 1, 40), (32, 4, 128, 128, 17, 50),
    (24, 8, 64, 64, 20, 60), (12, 4, 64, 64, 50, 90)])
@pytest.mark.parametrize("dtype,atol", [(torch.float16, 4e-3), (torch.bfloat16, 3.2e-2)])
def test_tiled_attention_matches_the_per_token_kernel(heads, kv_heads, dim, vdim, window, n, dtype, atol):
    """The matrix-core kernel (tiles of 16 queries, portions cut at odd places, a decoded token as a tile of one) against
    the per-token kernel on the same 16-bit inputs: they differ by rounding only."""
    cuts = [0, 5, 5 + 37, n - 1, n] if n > 45 else [0, 3, n - 1, n]
    for cap in (7.0, None):
        kw = dict(softcap=cap, seed=n + heads, dtype=dtype, cuts=cuts)
        tiled, want = _attention_case(heads, kv_heads, dim, vdim, window, n, tiled=True, **kw)
        plain, _ = _attention_case(heads, kv_heads, dim, vdim, window, n, tiled=False, **kw)
        assert (tiled - plain).abs().max() < atol * max(1.0, float(plain.abs().max()))
        assert (tiled - want).abs().max() < 0.3     # (16-bit q and k after their norms: uncapped scores reach +-45)


@pytest.mark.parametrize("window,n", [(9, 60), (16, 70), (37, 150), (64, 131)])
def test_tiled_window_edges_show_in_the_output(window, n):
    for qi in (n - 1, n - 2, 48 if n > 48 + 1 else n - 3, 17):
        for back in (window - 1, window):
            kj = qi - back
            if kj < 0:
                continue
            args = (4, 2, 64, 64, window, n, 30.0)
            kw = dict(seed=qi * 7 + back, standout=(qi, kj), dtype=torch.float16, cuts=[0, n - 1, n])
            got, want = _attention_case(*args, tiled=True, **kw)
            assert (got - want).abs().max() < 2e-2, (qi, kj)


@pytest.mark.parametrize("window,n", [(9, 60), (16, 70), (37, 150), (64, 131)])
def test_window_edges_show_in_the_output(window, n):
    """A key whose score dominates, placed just inside and just outside the window of the last prompt token, of the decoded
    token, and of a token at a block border: leaving it out (or letting it in) changes the output by O(1)."""
    for qi in (n - 1, n - 2, 48 if n > 48 + 1 else n - 3):
        for back in (window - 1, window):       # last visible key, first hidden key
            kj = qi - back
            if kj < 0:
                continue
            got, want = _attention_case(4, 2, 16, 16, window, n, 30.0, seed=qi * 7 + back, standout=(qi, kj))
            assert (got - want).abs().max() < 5e-5, (qi, kj)


# ---- the model ----------------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def default_case():
    cfg = O.make_config(layers=[O.attention_layer(mlp=O.dense_mlp(96)), O.attention_layer(mlp=O.moe_mlp(48, 5, 2)),
                                O.attention_layer(heads=2, kv_heads=1, dim=32, vdim=16, window=20, mlp=O.dense_mlp(64))],
                        loop=(1, 3, 2))
    W = O.random_weights(cfg, seed=3)
    toks = tokens_for(cfg, 75, 11)
    trace = []
    want = O.forward(cfg, W, toks, trace)
    return cfg, W, toks, want, trace


@pytest.mark.parametrize("dtype,tol", [("float32", F32_TOL), ("bfloat16", BF16_TOL)])
def test_whole_prompt_logits_and_every_layer_run(tmp_path, default_case, dtype, tol):
    cfg, W, toks, want, trace = default_case
    model = make_model(tmp_path / "m", cfg, W, dtype)
    model.layer_tap = []
    got = model.step([entry(2, toks, 0)])
    assert len(model.layer_tap) == len(trace) == 1 + 2 * 2
    for i, (a, b) in enumerate(zip(model.layer_tap, trace)):
        assert rel_err(a, b) < tol, f"layer run {i}"
    assert rel_err(got, want) < tol
    # the fused step (no tap) computes the same stream
    model.layer_tap = None
    model.free_seqs_resources([2])
    again = model.step([entry(0, toks, 0)])
    assert rel_err(again, got) < 1e-6 if dtype == "float32" else rel_err(again, got) < 1e-2


@pytest.mark.parametrize("dtype,tol", [("float32", F32_TOL), ("bfloat16", BF16_TOL)])
def test_decoding_and_portions_match_the_whole_prompt(tmp_path, default_case, dtype, tol):
    cfg, W, toks, want, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, dtype)
    # token by token from the first token on (the first tokens of a sequence, long decoding past every window)
    rows = [model.step([entry(1, toks[i:i + 1], i)]) for i in range(len(toks))]
    assert rel_err(torch.cat(rows), want) < tol
    model.free_seqs_resources([1])
    # portions of changing size, down to two tokens and one, cut inside blocks and windows
    for sizes in ([2, 2, 3, 9, 16, 1, 17, 2, 23], [31, 2, 5, 1, 1, 30, 5], [16, 16, 16, 16, 11]):
        at, rows = 0, []
        for n in sizes:
            rows.append(model.step([entry(3, toks[at:at + n], at)]))
            at += n
        assert at == len(toks)
        assert rel_err(torch.cat(rows), want) < tol, sizes
        model.free_seqs_resources([3])


def test_decode_graph_replays_match_eager_steps(tmp_path, default_case):
    """Pure-decode steps replay a captured hipGraph: several replays, with eager prompt portions and a changing batch in
    between, every one against the oracle."""
    cfg, W, toks, want, _ = default_case
    from swiftllm_amd import EngineConfig, build_model
    path = write_model(tmp_path / "g", cfg, W)
    ecfg = EngineConfig(model_path=path, use_dummy=False, block_size=16, gpu_mem_utilization=0.9, num_cpu_blocks=0,
                        max_seqs_in_block_table=4, max_blocks_per_seq=16, max_batch_size=4, max_tokens_in_batch=256,
                        dtype="float32", use_hip_graph=True)
    model = build_model(ecfg)
    model.load_weights()
    model.init_kvcache_and_swap(24)
    other = tokens_for(cfg, 60, 31)
    want2 = O.forward(cfg, W, other)
    model.step([entry(0, toks[:20], 0, want=[])])
    got0, got1 = [], []
    for i in range(20, 30):         # batch 1: one capture, ten replays
        got0.append(model.step([entry(0, toks[i:i + 1], i)]).clone())
    model.step([entry(1, other[:33], 0, want=[])])      # an eager portion in between
    for i in range(12):             # batch 2: another capture
        out = model.step([entry(0, toks[30 + i:31 + i], 30 + i), entry(1, other[33 + i:34 + i], 33 + i)])
        got0.append(out[:1].clone())
        got1.append(out[1:].clone())
    assert model.graph_captures == 2
    assert rel_err(torch.cat(got0), want[20:42]) < F32_TOL
    assert rel_err(torch.cat(got1), want2[33:45]) < F32_TOL


def test_unequal_batches_and_reused_blocks_and_rows(tmp_path, default_case):
    cfg, W, toks, want, _ = default_case
    seqs = {0: toks, 1: tokens_for(cfg, 40, 5), 2: tokens_for(cfg, 9, 6), 3: tokens_for(cfg, 58, 7)}
    wants = {0: want, **{k: O.forward(cfg, W, v) for k, v in seqs.items() if k}}
    # a pool that cannot hold all four at once: 75 + 40 + 58 tokens need 5 + 3 + 4 blocks
    model = make_model(tmp_path / "m", cfg, W, "float32", num_blocks=12)
    got = {k: [] for k in seqs}
    at = {k: 0 for k in seqs}
    # sequences 0, 1, 2 interleaved: portions of one beside single tokens of another
    plan = [[(0, 30), (1, 1), (2, 2)], [(0, 1), (1, 17), (2, 7)], [(0, 2), (1, 1)], [(1, 21), (0, 1)], [(0, 41)]]
    for step in plan:
        es = [entry(k, seqs[k][at[k]:at[k] + n], at[k]) for k, n in step]
        out = model.step(es)
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n])
            o += n
            at[k] += n
    for k in (0, 1, 2):
        assert at[k] == len(seqs[k])
        assert rel_err(torch.cat(got[k]), wants[k]) < F32_TOL, k
    # rows 1 and 2 end; their blocks and row 1 are used again by another request beside row 0's decoding
    model.free_seqs_resources([1, 2])
    free_before = model.gpu_block_manager.num_free_blocks
    out = model.step([entry(1, seqs[3][:50], 0)])
    assert model.gpu_block_manager.num_free_blocks == free_before - 4
    rest = model.step([entry(1, seqs[3][50:], 50)])
    assert rel_err(torch.cat((out, rest)), wants[3]) < F32_TOL
    # ... and row 0, untouched by all that, still decodes correctly: one more token against a longer oracle run
    longer = toks + [7]
    w2 = O.forward(cfg, W, longer)
    assert rel_err(model.step([entry(0, [7], len(toks))]), w2[-1:]) < F32_TOL


@pytest.mark.parametrize("dtype,tol", [("float32", F32_TOL), ("bfloat16", BF16_TOL)])
def test_other_sizes(tmp_path, dtype, tol):
    cfg = varied_config()
    W = O.random_weights(cfg, seed=9)
    toks = tokens_for(cfg, 90, 2)
    trace = []
    want = O.forward(cfg, W, toks, trace)
    model = make_model(tmp_path / "m", cfg, W, dtype)
    model.layer_tap = []
    got = model.step([entry(0, toks[:41], 0)])
    assert len(model.layer_tap) == len(trace) == 2 * 2 + 2
    model.layer_tap = None
    got = torch.cat([got] + [model.step([entry(0, toks[i:i + 1], i)]) for i in range(41, 90)])
    if dtype == "float32":
        assert rel_err(got, want) < tol
    else:
        # bfloat16 inputs can flip a top-1 routing decision that the float64 oracle makes by a hair, and such a token is
        # then legitimately far off: most positions must agree, and the fp32 run above pins the arithmetic
        errs = torch.tensor([rel_err(got[i:i + 1], want[i:i + 1]) for i in range(got.shape[0])])
        assert float((errs < tol).float().mean()) >= 0.7, errs


def test_matrix_core_paths_in_the_model(tmp_path):
    """Head sizes the matrix-core attention serves and expert widths the matrix-core expert products serve, in bfloat16:
    whole prompt (tiles of 16 queries, experts through sorted library products), portions, and decoding (tiles of one query
    with shared-out pages, expert-stationary products) against the oracle; and the per-token kernels on the same model."""
    from swiftllm_amd.worker.kernels import window_attn
    layers = [O.attention_layer(heads=4, kv_heads=2, dim=64, vdim=64, window=44, mlp=O.moe_mlp(32, 4, 2)),
              O.attention_layer(heads=2, kv_heads=1, dim=128, vdim=64, window=24, mlp=O.dense_mlp(128))]
    cfg = O.make_config(width=128, vocab=96, layers=layers, loop=(0, 2, 2), max_positions=256)
    W = O.random_weights(cfg, seed=21)
    toks = tokens_for(cfg, 150, 4)
    want = O.forward(cfg, W, toks)
    model = make_model(tmp_path / "m", cfg, W, "bfloat16")
    assert window_attn.tiles_supported(model.model_config.layers[0].mixer, torch.bfloat16)

    def run(seq):
        out = [model.step([entry(seq, toks[:100], 0)]), model.step([entry(seq, toks[100:131], 100)])]
        out += [model.step([entry(seq, toks[i:i + 1], i)]) for i in range(131, 150)]
        return torch.cat(out)

    tiled = run(0)
    saved = window_attn.TILES_MIN_TOKENS
    window_attn.TILES_MIN_TOKENS = 1 << 30
    try:
        plain = run(1)
    finally:
        window_attn.TILES_MIN_TOKENS = saved
    for got in (tiled, plain):
        errs = torch.tensor([rel_err(got[i:i + 1], want[i:i + 1]) for i in range(got.shape[0])])
        assert float((errs < BF16_TOL).float().mean()) >= 0.9, errs
    errs = torch.tensor([rel_err(tiled[i:i + 1], plain[i:i + 1]) for i in range(tiled.shape[0])])
    assert float((errs < BF16_TOL).float().mean()) >= 0.9, errs


def test_no_loop_and_single_pass_loop(tmp_path):
    layers = [O.attention_layer(mlp=O.dense_mlp(32)), O.attention_layer(mlp=O.moe_mlp(16, 4, 2))]
    for name, loop in (("a", None), ("b", (1, 2, 1)), ("c", (0, 2, 3))):
        cfg = O.make_config(width=32, vocab=50, layers=layers, loop=loop, max_positions=64)
        W = O.random_weights(cfg, seed=4)
        toks = tokens_for(cfg, 30, 8)
        model = make_model(tmp_path / name, cfg, W, "float32")
        assert rel_err(model.step([entry(0, toks, 0)]), O.forward(cfg, W, toks)) < F32_TOL, loop


def test_far_token_reaches_the_logits_through_the_depth(tmp_path):
    """With windows much shorter than the prompt, a change of the FIRST token reaches the last position only through the
    stack's depth (looped layers included); both implementations must agree on how much."""
    layers = [O.attention_layer(window=12, mlp=O.dense_mlp(64)), O.attention_layer(window=12, mlp=O.dense_mlp(64))]
    cfg = O.make_config(layers=layers, loop=(0, 2, 4), max_positions=128)
    W = O.random_weights(cfg, seed=12)
    toks = tokens_for(cfg, 80, 3)
    other = [(toks[0] + 1) % cfg["vocab"]] + toks[1:]
    model = make_model(tmp_path / "m", cfg, W, "float32")
    a = model.step([entry(0, toks, 0, want=[79])])
    b = model.step([entry(1, other, 0, want=[79])])
    wa, wb = O.forward(cfg, W, toks)[-1:], O.forward(cfg, W, other)[-1:]
    assert rel_err(a, wa) < F32_TOL and rel_err(b, wb) < F32_TOL
    assert rel_err(a.double().cpu() - b.double().cpu(), wa - wb) < 1e-2 or (wa - wb).abs().max() < 1e-6


def test_swap_out_and_in_keeps_the_sequence(tmp_path, default_case):
    cfg, W, toks, want, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, "float32", num_blocks=12, cpu_blocks=8)
    first = model.step([entry(0, toks[:40], 0)])
    model.swap_out_seqs([0])
    assert model.gpu_block_manager.num_free_blocks == 12
    model.step([entry(1, tokens_for(cfg, 100, 1), 0, want=[])])      # overwrites the freed blocks
    model.free_seqs_resources([1])
    model.step([entry(2, tokens_for(cfg, 30, 2), 0, want=[])])
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
    ecfg = EngineConfig(model_path=path, use_dummy=False, block_size=16, gpu_mem_utilization=0.05, num_cpu_blocks=8,
                        max_seqs_in_block_table=4, max_blocks_per_seq=16, max_batch_size=4, max_tokens_in_batch=256,
                        dtype="float32", use_hip_graph=False)
    prompts = [tokens_for(cfg, n, 20 + n) for n in (5, 33, 18)]
    outs = (6, 12, 9)

    def oracle(prompt, n):
        seq = list(prompt)
        for _ in range(n):
            lg = O.forward(cfg, W, seq)[-1]
            top2 = torch.topk(lg, 2).values
            assert float(top2[0] - top2[1]) > 1e-4, "the test's weights make a close call"
            seq.append(int(torch.argmax(lg)))
        return seq[len(prompt):]

    async def run():
        engine = Engine(ecfg)
        await engine.initialize()
        assert type(engine.model).__name__ == "KekapelModel"
        loops = asyncio.ensure_future(engine.start_all_event_loops())
        res = await asyncio.gather(*[engine.add_request_and_wait(RawRequest("", n, p)) for p, n in zip(prompts, outs)])
        loops.cancel()
        try:
            await loops
        except (asyncio.CancelledError, Exception):
            pass
        return [r[1] for r in res]

    got = asyncio.run(run())
    for g, p, n in zip(got, prompts, outs):
        assert g == oracle(p, n)
