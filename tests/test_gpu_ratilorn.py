"""Ratilorn on the GPU against the plain implementation in tests/ratilorn_oracle.py: every mechanism alone, whole prompts,
token-by-token decoding, portions down to two tokens, unequal batches, reused blocks and state slots, far keys and page
borders, the first tokens of a sequence, long decoding, odd sizes, hipGraph replays, swapping, and greedy generation through
the Engine and its scheduler. Configurations and weights are made here (small, random, seeded)."""
import asyncio
import random

import pytest
import torch

import ratilorn_oracle as O

pytestmark = pytest.mark.gpu

F32_TOL = 3e-5      # relative rms error of fp32 logits (true fp32 products, fp32 statistics)
BF16_TOL = 8e-2     # the same in bfloat16 (bf16 products and activations, fp32 stream, statistics and recurrences)
EPS = 1e-5


def f64(W):
    return {k: v.double() for k, v in W.items()}


def make_model(path, cfg, W, dtype="float32", num_blocks=48, max_seqs=4, cpu_blocks=0, graph=False):
    from swiftllm_amd import EngineConfig, build_model
    O.write_checkpoint(str(path), cfg, W)
    ecfg = EngineConfig(model_path=str(path), use_dummy=False, block_size=16, gpu_mem_utilization=0.9,
                        num_cpu_blocks=cpu_blocks, max_seqs_in_block_table=max_seqs,
                        max_blocks_per_seq=-(-cfg["max_positions"] // 16), max_batch_size=max_seqs,
                        max_tokens_in_batch=1024, dtype=dtype, use_hip_graph=graph)
    model = build_model(ecfg)
    model.load_weights()
    model.init_kvcache_and_swap(num_blocks)
    return model


def row_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def rel_err(got, want):
    return float(row_err(got, want).max())


def close(got, want, dtype, tol=None):
    """fp32 runs are held to the tolerance everywhere; 16-bit runs at the median and at most positions (rounding moves a
    router's close calls, and a token that goes to another expert differs by more than rounding)."""
    e = row_err(got, want)
    if dtype in ("float32", torch.float32):
        return float(e.max()) < (tol or F32_TOL)
    tol = tol or BF16_TOL
    return float(e.median()) < tol / 2 and float((e < tol).double().mean()) >= 0.75


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


def i32(xs):
    return torch.tensor(xs, dtype=torch.int32, device="cuda")


class Pool:
    """A block pool with a shuffled block table and the per-token arrays of hand-made steps, for the attention kernels."""

    def __init__(self, mixer, dtype, max_len, rows=3, seed=0):
        from swiftllm_amd.worker.kernels.window_attn import PoolSlice
        per_seq = -(-max_len // 16)
        ids = list(range(rows * per_seq + 5))
        random.Random(seed).shuffle(ids)
        self.table = i32(ids[:rows * per_seq]).view(rows, per_seq).contiguous()
        pad = 24        # the slices do not start at the block's first element
        self.slice = PoolSlice(pad, pad + mixer.k_size * 16)
        elems = pad + (mixer.k_size + mixer.v_size) * 16 + 8
        # (slots that were never written hold a large finite number: a masked key's value is multiplied by a zero weight)
        self.pool = torch.full((len(ids), elems), 777.0, dtype=dtype, device="cuda")

    @staticmethod
    def step(portions):
        """portions: [(row, start, count)] -> tok_seq, tok_pos, (tile_row0, tile_cnt)"""
        seq = [p[0] for p in portions for _ in range(p[2])]
        pos = [p[1] + j for p in portions for j in range(p[2])]
        row0, cnt, at = [], [], 0
        for p in portions:
            for s in range(0, p[2], 16):
                row0.append(at + s)
                cnt.append(min(16, p[2] - s))
            at += p[2]
        return i32(seq), i32(pos), (i32(row0), i32(cnt))


class Slots:
    """A StateSlotManager and the per-token arrays of hand-made steps, for the kernels that carry state."""

    def __init__(self, floats, num_slots=3):
        from swiftllm_amd.worker.state_slots import StateSlotManager
        self.mgr = StateSlotManager(num_slots)
        self.off = [self.mgr.add_region(f) for f in floats]
        self.mgr.allocate()
        self.mgr.pool.fill_(float("nan"))       # nothing may be read before it is written

    def ref(self, portions):
        from swiftllm_amd.worker.kernels.rms_stream import StateRef
        codes = self.mgr.begin_step([p[0] for p in portions], [p[1] for p in portions])
        pos = [p[1] + j for p in portions for j in range(p[2])]
        start = [p[1] for p in portions for _ in range(p[2])]
        state = [int(c) for p, c in zip(portions, codes) for _ in range(p[2])]
        seq = [p[0] for p in portions for _ in range(p[2])]
        cnt = [p[2] for p in portions]
        row0 = [sum(cnt[:i]) for i in range(len(cnt))]
        return StateRef(self.mgr.pool, i32(pos), i32(start), i32(state), i32(seq), i32(row0), i32(cnt))


def cut(n, sizes):
    """[(start, count)] of a sequence of n tokens cut into portions of the given sizes (the last repeats)."""
    out, at, i = [], 0, 0
    while at < n:
        c = min(sizes[min(i, len(sizes) - 1)], n - at)
        out.append((at, c))
        at += c
        i += 1
    return out


# ---- mechanisms alone ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_stream_step_with_the_norm_on_the_result(dtype):
    from swiftllm_amd.worker.kernels.rms_stream import post_norm_add
    g = torch.Generator().manual_seed(0)
    n, w = 37, 72
    x0 = torch.randn(n, w, generator=g) * 2 + 0.5
    a, b = (torch.randn(n, w, generator=g) * 3).to(dtype), torch.randn(n, w, generator=g).to(dtype)
    post, wa, wb, pre = [1 + 0.3 * torch.randn(w, generator=g) for _ in range(4)]
    ad, bd = a.double(), b.double()
    cases = {
        "one result": (dict(b=None), ad),
        "two results normed apart and averaged": (dict(b=b, a_norm=wa, b_norm=wb, coef=0.5),
                                                  0.5 * (O.unit_rms(ad, EPS) * wa + O.unit_rms(bd, EPS) * wb)),
        "two addends as they are": (dict(b=b), ad + bd),
    }
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    for name, (kw, y) in cases.items():
        want_x = x0.double() + O.unit_rms(y, EPS) * post
        for with_pre in (False, True):
            x = x0.clone().cuda()
            kw_dev = {k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in kw.items()}
            out = post_norm_add(x, a.cuda(), post.cuda(), eps=EPS, pre=pre.cuda() if with_pre else None, **kw_dev)
            assert (x.cpu().double() - want_x).abs().max() < 2e-5, name
            want_out = O.unit_rms(want_x, EPS) * pre if with_pre else want_x
            assert (out.cpu().double() - want_out).abs().max() < tol * float(want_out.abs().max()), name
        x = x0.clone().cuda()
        assert post_norm_add(x, a.cuda(), post.cuda(), eps=EPS, want_out=False,
                             **{k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in kw.items()}) is None
        assert (x.cpu().double() - want_x).abs().max() < 2e-5


def _attention_weights(H, G, d, e, width, seed, sigmoid):
    mx = {"heads": H, "kv_heads": G, "dim": d, "vdim": e, "scale": 1.7 * d ** -0.5, "v_mix": True}
    cfg = O.make_config(layers=[{"type": "attention", "mixer": mx, "mlp": None}] if sigmoid else
                        [{"type": "parallel", "mlp": None,
                          "mixer": {"left": mx, "right": {"heads": 1, "vdim": 8, "state": 8, "groups": 1, "conv": 2,
                                                         "norm_groups": 1}}}], width=width)
    return mx, O.random_weights(cfg, seed)


def _run_attention(mx, W, p, h, v_other, lam, dtype, sigmoid, portions_of, tiled, window=0):
    """The framework's side of one attention mixer without its projections' library products: bias / norm / blend / store,
    then the attention over the pool, for sequences fed in the given portions. -> per sequence [T, heads * vdim]."""
    from swiftllm_amd.model_config import RatilornAttentionConfig
    from swiftllm_amd.worker.kernels.sigmoid_attn import sigmoid_attention
    from swiftllm_amd.worker.kernels.window_attn import AttentionSpec, masked_attention, qkv_bias_norm_store
    mixer = RatilornAttentionConfig(mx, sigmoid=sigmoid)
    mixer.window = window       # (an argument of the kernels; the design itself sees every earlier key)
    dev = lambda name: W[p + name].float().cuda().contiguous()
    wqkv = torch.cat((W[p + "q"], W[p + "k"], W[p + "v"]), dim=0)
    lens = [x.shape[0] for x in h]
    pool = Pool(mixer, dtype, max(lens), rows=len(h))
    outs = [[] for _ in h]
    steps = max(len(c) for c in portions_of)
    for s in range(steps):
        batch = [(i, *portions_of[i][s]) for i in range(len(h)) if s < len(portions_of[i])]
        rows = torch.cat([h[i][a:a + c] for i, a, c in batch])
        qkv = torch.cat(((rows.double() @ wqkv.double().T).float(), torch.zeros(rows.shape[0], 8)), dim=1).to(dtype).cuda()
        other = None
        if v_other is not None:
            other = torch.cat([v_other[i][a:a + c] for i, a, c in batch]).to(dtype).cuda()
        tok_seq, tok_pos, tiles = Pool.step(batch)
        qkv_bias_norm_store(qkv, dev("q.b"), dev("k.b"), dev("v.b"), None if sigmoid else dev("q.norm"),
                            None if sigmoid else dev("k.norm"), pool.pool, pool.slice, pool.table, tok_seq, tok_pos, mixer,
                            EPS, other, lam)
        if sigmoid:
            o = sigmoid_attention(qkv, pool.pool, pool.slice, pool.table, tok_seq, tok_pos, mixer, dev("talk"), dev("r1"),
                                  dev("r2"), dev("pb"), tiles if tiled else None, 4096)
        else:
            spec = AttentionSpec(mixer.num_q_heads, mixer.num_kv_heads, mixer.head_dim, mixer.value_dim, mixer.scale)
            o = masked_attention(qkv, pool.pool, pool.slice, pool.table, tok_seq, tok_pos, spec, tiles if tiled else None, 4096)
        at = 0
        for i, a, c in batch:
            outs[i].append(o[at:at + c].float().cpu())
            at += c
    return [torch.cat(o) for o in outs]


def _check_attention(H, G, d, e, lens, dtype, sigmoid, tiled, sizes=((1000,),), blend=False, seed=0, tune=None):
    width = 24
    mx, W = _attention_weights(H, G, d, e, width, seed, sigmoid)
    p = "l0.mix." if sigmoid else "l0.mix.left."
    if tune:
        tune(W, p)
    g = torch.Generator().manual_seed(seed + 1)
    h = [torch.randn(n, width, generator=g).to(dtype).float() for n in lens]
    v_other = [torch.randn(n, G * e, generator=g).to(dtype).float() for n in lens] if blend else None
    lam = float(W[p + "vmix"]) if blend else 0.0
    Wd = f64(W)
    Wd[p + "o"] = torch.eye(H * e, dtype=torch.float64)       # the oracle's mixer output is then the attention's own
    want = []
    for i, x in enumerate(h):
        if sigmoid:
            want.append(O.sigmoid_attention(x.double(), Wd, p, mx, EPS, v_other[i].double() if blend else None)[0])
        else:
            want.append(O.softmax_attention(x.double(), Wd, p, mx, EPS))
    for sz in sizes:
        got = _run_attention(mx, W, p, h, v_other, lam, dtype, sigmoid, [cut(n, sz) for n in lens], tiled)
        for gi, wi in zip(got, want):
            scale = float(wi.abs().max())
            tol = 3e-5 if dtype == torch.float32 else 3e-2
            assert float((gi.double() - wi).abs().max()) < tol * scale, (sz, float((gi.double() - wi).abs().max()), scale)
    return want


@pytest.mark.parametrize("H,G,d,e,lens", [(4, 2, 16, 24, (150, 37)), (3, 1, 40, 8, (70,)), (2, 2, 8, 8, (1, 2)),
                                          (5, 5, 32, 16, (45, 17, 64)), (8, 4, 64, 32, (100,))])
def test_sigmoid_attention_fp32(H, G, d, e, lens):
    _check_attention(H, G, d, e, lens, torch.float32, True, False, sizes=((1000,), (7, 1, 2, 16, 1), (1,)), blend=True)


@pytest.mark.parametrize("H,G,d,e,lens", [(8, 4, 64, 32, (150, 37)), (4, 1, 64, 64, (70,)), (6, 3, 32, 32, (1, 2, 33)),
                                          (16, 4, 128, 128, (64,)), (3, 3, 96, 96, (49,)), (20, 4, 48, 48, (40,)),
                                          (32, 8, 128, 128, (40,))])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_sigmoid_attention_on_the_matrix_core(H, G, d, e, lens, dtype):
    from swiftllm_amd.model_config import RatilornAttentionConfig
    from swiftllm_amd.worker.kernels.sigmoid_attn import tiles_supported
    assert tiles_supported(RatilornAttentionConfig({"heads": H, "kv_heads": G, "dim": d, "vdim": e, "scale": 1.0}, True), dtype)
    _check_attention(H, G, d, e, lens, dtype, True, True, sizes=((1000,), (7, 1, 2, 16, 1), (1,)), blend=True)


@pytest.mark.parametrize("far", [13, 15, 16, 271, 272])      # inside a page, on both sides of a page border, near and far
@pytest.mark.parametrize("dtype,tiled,d", [(torch.float32, False, 24), (torch.bfloat16, True, 64), (torch.bfloat16, False, 24)])
def test_a_far_key_among_hundreds_is_found(dtype, tiled, d, far):
    """Every key but one is pushed far below the sigmoid's threshold; the one that stands out lies hundreds of positions back,
    beyond many page borders, and the distance term takes its full toll. Leaving it out would change the last rows entirely."""
    def tune(W, p):
        W[p + "pb"].fill_(-9.0)
        W[p + "r1"].fill_(0.5)
        W[p + "r2"].fill_(0.25)
        for nm in ("q", "k"):
            W[p + nm].zero_()
            W[p + nm + ".b"].zero_()
    n = 420
    mx, W = _attention_weights(2, 1, d, 16, 24, 5, True)
    p = "l0.mix."
    tune(W, p)
    # queries are zero but at the last tokens, keys are zero but at the far token: that one pair scores scale * dim, all
    # others zero
    g = torch.Generator().manual_seed(9)
    h = torch.randn(n, 24, generator=g).to(torch.bfloat16).float() * 0.1
    h[:, :2] = 0
    h[far, 1] = 1.0
    h[-3:, 0] = 1.0
    W[p + "q"][:, 0] = 8.0
    W[p + "k"][:, 1] = 8.0
    mx["scale"] = 14.0 / d
    Wd = f64(W)
    Wd[p + "o"] = torch.eye(2 * 16, dtype=torch.float64)
    want = O.sigmoid_attention(h.double(), Wd, p, mx, EPS)[0]
    shown = want[-1].abs().max()
    h2 = h.clone()
    h2[far, 1] = 0
    without = O.sigmoid_attention(h2.double(), Wd, p, mx, EPS)[0]
    assert float((want[-1] - without[-1]).abs().max()) > 0.3 * float(shown), "the test's weights do not show the far key"
    for sizes in ((1000,), (n - 3, 1)):
        got = _run_attention(mx, W, p, [h], None, 0.0, dtype, True, [cut(n, sizes)], tiled)[0]
        tol = 3e-5 if dtype == torch.float32 else 3e-2
        assert float((got[-3:].double() - want[-3:]).abs().max()) < tol * float(shown)


@pytest.mark.parametrize("dtype,tiled,d,window", [(torch.float32, False, 24, 21), (torch.bfloat16, True, 64, 21),
                                                  (torch.bfloat16, True, 32, 16), (torch.float32, False, 8, 1)])
def test_sigmoid_attention_inside_a_window(dtype, tiled, d, window):
    """The kernels' window argument: query i sees keys i - window + 1 .. i. Scores depend on positions through i - j only, so
    the plain evaluation of the last `window` tokens alone gives query i's row. The key just inside the window and the one
    just outside are made to stand out: one key more or less changes the row by several times the tolerance."""
    n = 70
    mx, W = _attention_weights(4, 2, d, 16, 24, 11, True)
    p = "l0.mix."
    W[p + "pb"].fill_(-6.0)
    for nm in ("q", "k"):
        W[p + nm].zero_()
        W[p + nm + ".b"].zero_()
    W[p + "q"][:, 0] = 8.0
    W[p + "k"][:, 1] = 8.0
    mx["scale"] = 12.0 / d
    g = torch.Generator().manual_seed(4)
    h = torch.randn(n, 24, generator=g).to(torch.bfloat16).float() * 0.1
    h[:, :2] = 0
    h[:, 0] = 1.0               # every query looks for the marked keys
    h[::3, 1] = 1.0             # every third token is one: the window's edge passes over them
    Wd = f64(W)
    Wd[p + "o"] = torch.eye(4 * 16, dtype=torch.float64)
    want = torch.stack([O.sigmoid_attention(h[max(0, i - window + 1):i + 1].double(), Wd, p, mx, EPS)[0][-1] for i in range(n)])
    wider = torch.stack([O.sigmoid_attention(h[max(0, i - window):i + 1].double(), Wd, p, mx, EPS)[0][-1] for i in range(n)])
    assert float((want - wider).abs().max()) > 0.1 * float(want.abs().max()), "the test's weights do not show the edge"
    tol = 3e-5 if dtype == torch.float32 else 3e-2
    for sizes in ((1000,), (33, 1), (5, 2, 16)):
        got = _run_attention(mx, W, p, [h], None, 0.0, dtype, True, [cut(n, sizes)], tiled, window=window)[0]
        assert float((got.double() - want).abs().max()) < tol * float(want.abs().max()), sizes


@pytest.mark.parametrize("H,G,d,e,lens,dtype,tiled", [(4, 2, 16, 24, (150, 37), torch.float32, False),
                                                       (6, 3, 96, 96, (70, 16), torch.bfloat16, True),
                                                       (3, 1, 40, 8, (33,), torch.bfloat16, False)])
def test_softmax_attention_with_biases_and_weighted_norm(H, G, d, e, lens, dtype, tiled):
    _check_attention(H, G, d, e, lens, dtype, False, tiled, sizes=((1000,), (5, 1, 2, 16, 1)))


@pytest.mark.parametrize("heads,P,N,groups,conv,parts,lens", [(3, 8, 12, 1, 3, 1, (70, 9)), (4, 24, 20, 2, 1, 2, (33,)),
                                                             (2, 32, 48, 2, 4, 1, (40, 1, 2)), (6, 16, 128, 3, 2, 3, (21,)),
                                                             (1, 64, 16, 1, 5, 4, (50,)), (2, 8, 256, 1, 2, 1, (37,))])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_state_space_mixer_in_portions_and_reused_slots(heads, P, N, groups, conv, parts, lens, dtype):
    from swiftllm_amd.model_config import StateSpaceConfig
    from swiftllm_amd.worker.kernels.ssd import state_space_mixer
    width = 24
    rt = {"heads": heads, "vdim": P, "state": N, "groups": groups, "conv": conv, "norm_groups": parts}
    cfg = O.make_config(layers=[{"type": "parallel", "mlp": None, "mixer": {
        "left": {"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 1.0}, "right": rt}}], width=width)
    W = O.random_weights(cfg, 2)
    p = "l0.mix.right."
    mixer = StateSpaceConfig(rt)
    g = torch.Generator().manual_seed(3)
    h = [torch.randn(n, width, generator=g).to(dtype).float() for n in lens]
    Wd = f64(W)
    Wd[p + "o"] = torch.eye(mixer.inner, dtype=torch.float64)
    want = [O.state_space_mixer(x.double(), Wd, p, rt, EPS) for x in h]
    dev = lambda name: W[p + name].float().cuda().contiguous()
    conv_w = W[p + "conv"].t().contiguous().cuda()
    for sizes in ((1000,), (1,), (2, 5, 1, 16, 3)):
        slots = Slots([2 * (conv - 1) * mixer.conv_channels, mixer.state_elems], num_slots=len(lens))
        portions_of = [cut(n, sizes) for n in lens]
        outs = [[] for _ in lens]
        for s in range(max(len(c) for c in portions_of)):
            batch = [(i, *portions_of[i][s]) for i in range(len(lens)) if s < len(portions_of[i])]
            rows = torch.cat([h[i][a:a + c] for i, a, c in batch])
            # (a column slice of a wider matrix, as inside the model's fused projection)
            proj = torch.cat((torch.zeros(rows.shape[0], 8), (rows.double() @ W[p + "in"].double().T).float()), dim=1)
            proj = proj.to(dtype).cuda()[:, 8:]
            st = slots.ref(batch)
            y = state_space_mixer(proj, conv_w, dev("conv.b"), dev("A_log"), dev("dt_bias"), dev("D"), dev("norm"), st,
                                  slots.off[0], slots.off[1], mixer, EPS)
            at = 0
            for i, a, c in batch:
                outs[i].append(y[at:at + c].float().cpu())
                at += c
        for o, w_ in zip(outs, want):
            tol = 1e-4 if dtype == torch.float32 else 4e-2
            assert float((torch.cat(o).double() - w_).abs().max()) < tol * float(w_.abs().max()), sizes
        slots.mgr.release(list(range(len(lens))))


@pytest.mark.parametrize("experts,top,groups", [(8, 2, (4, 2)), (16, 4, (4, 3)), (6, 1, (6, 2)), (12, 4, None), (9, 3, (3, 3)),
                                                (70, 5, (7, 3))])
def test_sigmoid_router_with_group_limited_choice(experts, top, groups):
    from swiftllm_amd.worker.kernels.moe import moe_route_grouped
    g = torch.Generator().manual_seed(experts)
    n, width = 200, 40
    h = torch.randn(n, width, generator=g)
    router = torch.randn(experts, width, generator=g) * 0.5
    # corrections that make most choice scores negative: masking an excluded expert with a zero would let it win
    corr = -0.8 + 0.4 * torch.randn(experts, generator=g)
    z = h.double() @ router.double().T
    idx, w = O.route(z, corr.double(), top, {"count": groups[0], "keep": groups[1]} if groups else None)
    assert float(((torch.sigmoid(z) + corr) < 0).double().mean()) > 0.3
    gi, gw = moe_route_grouped(h.cuda(), router.cuda(), corr.cuda(), top, groups[0] if groups else 1,
                               groups[1] if groups else 1)
    same = (gi.cpu().long() == idx).all(dim=-1)
    assert float(same.double().mean()) > 0.97        # (fp32 against float64: a close call may fall the other way)
    assert (gw.cpu().double()[same] - w[same]).abs().max() < 1e-5


@pytest.mark.parametrize("n", [23, 300])       # per-assignment kernels / assignments sorted by expert + library products
@pytest.mark.parametrize("experts,top,groups,shared", [(8, 2, (4, 2), 16), (5, 1, None, 0), (6, 6, (3, 3), 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixture_of_gated_units(experts, top, groups, shared, n, dtype):
    from swiftllm_amd.worker.layers.ratilorn_layer import RatilornFeedForward
    from swiftllm_amd.worker.ratilorn_weight import RatilornLayerWeight
    from swiftllm_amd.model_config import RatilornModelConfig
    from swiftllm_amd.worker.kernels.rms_stream import post_norm_add
    width = 32
    layer = O.attention_layer(mlp=O.moe_mlp(ff=16, experts=experts, top=top, groups=groups, shared=shared))
    cfg = O.make_config(layers=[layer], width=width)
    W = O.random_weights(cfg, 4)
    mcfg = RatilornModelConfig(cfg)
    lw = RatilornLayerWeight(0)
    lw.load(lambda name, shape: W[name].clone(), mcfg, mcfg.layers[0], dtype, torch.device("cuda"))
    ff = RatilornFeedForward(mcfg.layers[0], lw, False)
    g = torch.Generator().manual_seed(5)
    h = torch.randn(n, width, generator=g).to(dtype)
    a, b = ff.forward(h.cuda(), None, None)
    got = a.float() + (b.float() if b is not None else 0)
    want = O.moe_ff(h.double(), f64(W), "l0.mlp.", layer["mlp"])
    e = (got.cpu().double() - want).abs().max(dim=-1).values / want.abs().max()
    if dtype == torch.float32:
        assert float(e.max()) < 1e-5
    else:
        assert float(e.median()) < 2e-2 and float((e < 4e-2).double().mean()) > 0.9


# ---- the whole model -------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def default_case():
    cfg = O.make_config()
    W = O.random_weights(cfg, seed=3)
    toks = tokens_for(cfg, 90, 1)
    logits, streams = O.forward(f64(W), cfg, toks)
    return cfg, W, toks, logits, streams


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_logits_and_every_layer(tmp_path, default_case, dtype):
    cfg, W, toks, want, streams = default_case
    model = make_model(tmp_path / "m", cfg, W, dtype)
    assert type(model).__name__ == "RatilornModel"
    model.layer_tap = []
    got = model.step([entry(0, toks, 0)])
    assert len(model.layer_tap) == len(streams)
    for x, ref in zip(model.layer_tap, streams):
        if dtype == "float32":
            assert (x.cpu().double() - ref).abs().max() < 2e-4
        else:
            assert float((x.cpu().double() - ref).abs().median()) < 0.1
    assert close(got, want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_and_portions_match_the_whole_prompt(tmp_path, default_case, dtype):
    cfg, W, toks, want, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, dtype)
    assert close(run_in_portions(model, 0, toks, [1]), want, dtype)                     # token by token from the first
    assert close(run_in_portions(model, 1, toks, [2]), want, dtype)                     # pairs
    assert close(run_in_portions(model, 2, toks, [3, 2, 16, 1, 31, 2, 17, 1]), want, dtype)
    model.free_seqs_resources([0, 1, 2])
    assert close(run_in_portions(model, 0, toks, [58, 1]), want, dtype)                 # a prompt, then decoding
    if dtype == "bfloat16":     # the same positions whole and cut: the cut must not show beyond rounding
        whole = model.step([entry(1, toks, 0)])
        model.free_seqs_resources([1])
        parts = run_in_portions(model, 1, toks, [15, 2, 1, 33])
        assert float(row_err(parts, whole.float()).median()) < BF16_TOL / 2


def test_decode_graph_replays_match_eager_steps(tmp_path, default_case):
    cfg, W, toks, want, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, "float32", graph=True)
    other = tokens_for(cfg, 70, 2)
    want_other = O.forward(f64(W), cfg, other)[0]
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


def _serve(model, cfg, reqs, cuts, rows_total):
    """Up to rows_total live requests, portions beside decoded tokens, requests that sit steps out; finished requests give
    their blocks, block-table rows and state slots to new ones. -> the logits of every request."""
    lens = [len(r) for r in reqs]
    got = [[] for _ in reqs]
    at, k = [0] * len(reqs), [0] * len(reqs)
    waiting, live, rows = list(range(len(reqs))), {}, list(range(rows_total - 1, -1, -1))
    steps = 0
    while waiting or live:
        while waiting and rows:
            live[waiting.pop(0)] = rows.pop()
        batch, ended = [], []
        for r, row in live.items():
            if (steps + r) % 4 == 3 and len(live) > 1:
                continue
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
    return [torch.cat(g) for g in got]


def test_unequal_batches_and_reused_blocks_and_slots(tmp_path, default_case):
    cfg, W, _, _, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, "float32", num_blocks=20, max_seqs=4)
    lens = [70, 5, 33, 1, 48, 17, 2]
    reqs = [tokens_for(cfg, n, 50 + i) for i, n in enumerate(lens)]
    wants = [O.forward(f64(W), cfg, t)[0] for t in reqs]
    got = _serve(model, cfg, reqs, [[9, 1, 1, 30, 2], [2, 1], [33], [1], [16, 1], [3, 2], [1]], 4)
    assert model.gpu_block_manager.num_free_blocks == 20 and model.state.num_free_slots == 4
    for r in range(len(reqs)):
        assert rel_err(got[r], wants[r]) < F32_TOL, f"request {r}"


def varied_config():
    """Sizes that a symmetric configuration would hide: dim != vdim, heads not a power of two, one kv head, heads = kv heads,
    a layer without feed-forward, top = 1 and top = experts, no router groups, groups of one expert, no shared expert, a
    parallel layer first, a convolution of one tap, several state groups and norm parts, the first value-blending layer not
    the first attention layer, an attention layer that does not blend, a width that is no multiple of 8."""
    layers = [
        O.parallel_layer(heads=3, kv_heads=1, dim=24, vdim=8, s_heads=4, s_vdim=6, state=10, groups=2, conv=1, norm_groups=3,
                         scale=0.31,
                         mlp=O.moe_mlp(ff=12, experts=6, top=1, groups=(6, 2), shared=0)),
        O.attention_layer(heads=6, kv_heads=3, dim=16, vdim=8, v_mix=False, scale=0.4, mlp=None),
        O.attention_layer(heads=3, kv_heads=1, dim=24, vdim=24, v_mix=True, scale=0.11, mlp=O.dense_mlp(36)),
        O.parallel_layer(heads=2, kv_heads=2, dim=8, vdim=40, s_heads=1, s_vdim=20, state=33, groups=1, conv=5, norm_groups=1,
                         mlp=O.moe_mlp(ff=8, experts=3, top=3, groups=None, shared=20)),
        O.attention_layer(heads=2, kv_heads=2, dim=32, vdim=12, v_mix=True, mlp=O.moe_mlp(ff=16, experts=9, top=2,
                                                                                        groups=(3, 2), shared=4)),
    ]
    return O.make_config(layers=layers, width=44, vocab=37, max_positions=96, logit_scale=1.7)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_other_sizes(tmp_path, dtype):
    cfg = varied_config()
    W = O.random_weights(cfg, seed=5)
    toks = tokens_for(cfg, 75, 6)
    want, streams = O.forward(f64(W), cfg, toks)
    model = make_model(tmp_path / "m", cfg, W, dtype)
    model.layer_tap = []
    got = model.step([entry(0, toks, 0)])
    if dtype == "float32":
        for x, ref in zip(model.layer_tap, streams):
            assert (x.cpu().double() - ref).abs().max() < 2e-4
    model.layer_tap = None
    assert close(got, want, dtype)
    assert close(run_in_portions(model, 1, toks, [4, 1, 2, 17, 1]), want, dtype)


def random_config(rng):
    def mlp():
        kind = rng.choice(["dense", "moe", "moe", None])
        if kind == "dense":
            return O.dense_mlp(rng.choice([8, 24, 40]))
        if kind is None:
            return None
        count = rng.choice([1, 2, 3])
        per = rng.choice([1, 2, 4])
        keep = rng.randint(1, count)
        top = rng.randint(1, keep * per)
        return O.moe_mlp(ff=rng.choice([8, 16]), experts=count * per, top=top, groups=(count, keep) if rng.random() < 0.8 else None,
                         shared=rng.choice([0, 8]))
    vsize = rng.choice([16, 24, 48])
    layers = []
    for _ in range(rng.randint(2, 5)):
        if rng.random() < 0.5:
            G = rng.choice([g for g in (1, 2, 3) if vsize % g == 0])
            layers.append(O.attention_layer(heads=G * rng.choice([1, 2, 3]), kv_heads=G, dim=rng.choice([8, 16, 40]),
                                            vdim=vsize // G, v_mix=rng.random() < 0.8, mlp=mlp()))
        else:
            G = rng.choice([1, 2])
            groups = rng.choice([1, 2])
            layers.append(O.parallel_layer(heads=G * rng.choice([1, 2, 3]), kv_heads=G, dim=rng.choice([8, 16, 24]),
                                           vdim=rng.choice([8, 16]), s_heads=groups * rng.choice([1, 2]),
                                           s_vdim=rng.choice([4, 8, 20]), state=rng.choice([4, 16, 24]), groups=groups,
                                           conv=rng.randint(1, 4), norm_groups=rng.choice([1, 2]), mlp=mlp()))
    return O.make_config(layers=layers, width=rng.choice([24, 40, 56]), vocab=rng.choice([17, 50]), max_positions=80,
                         logit_scale=rng.choice([0.25, 1.0, 3.0]))


@pytest.mark.parametrize("seed", [1, 4, 8, 9])
def test_random_configurations_in_a_mixed_batch(tmp_path, seed):
    rng = random.Random(seed)
    cfg = random_config(rng)
    W = O.random_weights(cfg, seed=seed)
    model = make_model(tmp_path / "m", cfg, W, "float32", num_blocks=14, max_seqs=3)
    lens = [rng.randint(1, 70) for _ in range(5)]
    reqs = [tokens_for(cfg, n, seed * 10 + i) for i, n in enumerate(lens)]
    wants = [O.forward(f64(W), cfg, t)[0] for t in reqs]
    cuts = [[rng.choice([1, 2, 3, 16, 17, 40]) for _ in range(4)] + [1] for _ in reqs]
    got = _serve(model, cfg, reqs, cuts, 3)
    assert model.gpu_block_manager.num_free_blocks == 14
    for r in range(len(reqs)):
        assert rel_err(got[r], wants[r]) < F32_TOL, f"request {r} of {cfg['layers']}"


def test_matrix_core_paths_in_the_model(tmp_path):
    """Head sizes that the matrix-core attention kernels serve, in bfloat16: whole, in portions and decoded."""
    layers = [O.attention_layer(heads=8, kv_heads=4, dim=64, vdim=32, mlp=O.dense_mlp(64)),
              O.parallel_layer(heads=6, kv_heads=3, dim=96, vdim=96, s_heads=2, s_vdim=64, state=32, mlp=O.moe_mlp(32, 8, 2)),
              O.attention_layer(heads=4, kv_heads=2, dim=64, vdim=64, mlp=O.moe_mlp(32, 8, 2))]
    cfg = O.make_config(layers=layers, width=64, max_positions=320)
    W = O.random_weights(cfg, seed=7)
    toks = tokens_for(cfg, 300, 2)
    want = O.forward(f64(W), cfg, toks)[0]
    model = make_model(tmp_path / "m", cfg, W, "bfloat16")
    assert close(model.step([entry(0, toks, 0)]), want, "bfloat16")
    assert close(run_in_portions(model, 1, toks, [33, 2, 64, 1]), want, "bfloat16")


def test_first_tokens_of_a_sequence(tmp_path, default_case):
    """Sequences shorter than the convolution, alone and decoded, in blocks and slots that longer sequences used before."""
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
    W = O.random_weights(cfg, seed=8)
    toks = tokens_for(cfg, 330, 3)
    want = O.forward(f64(W), cfg, toks)[0]
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
    path = str(tmp_path / "m")
    O.write_checkpoint(path, cfg, W)
    ecfg = EngineConfig(model_path=path, use_dummy=False, block_size=16, gpu_mem_utilization=0.12, num_cpu_blocks=8,
                        max_seqs_in_block_table=4, max_blocks_per_seq=16, max_batch_size=4, max_tokens_in_batch=256,
                        dtype="float32", use_hip_graph=True)
    prompts = [tokens_for(cfg, n, 20 + n) for n in (5, 33, 18)]
    outs = (6, 12, 9)
    Wd = f64(W)

    def oracle(prompt, n):
        seq = list(prompt)
        for _ in range(n):
            lg = O.forward(Wd, cfg, seq)[0][-1]
            top2 = torch.topk(lg, 2).values
            assert float(top2[0] - top2[1]) > 1e-4, "the test's weights make a close call"
            seq.append(int(torch.argmax(lg)))
        return seq[len(prompt):]

    async def run():
        engine = Engine(ecfg)
        await engine.initialize()
        assert type(engine.model).__name__ == "RatilornModel"
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner_replays_a_mixed_schedule(tmp_path, dtype):
    """bin/trace_run as a user starts it: five requests through four block-table rows and state slots and a pool of 20 blocks,
    portions beside decoded tokens, a request that sits steps out, finished requests whose blocks and slot the next one takes."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = varied_config()
    W = O.random_weights(cfg, seed=13)
    path = str(tmp_path / "m")
    O.write_checkpoint(path, cfg, W)
    lens = {"a": 70, "b": 5, "c": 40, "d": 1, "e": 33}
    reqs = {k: tokens_for(cfg, n, 90 + i) for i, (k, n) in enumerate(lens.items())}
    schedule = [[("a", 30), ("b", 2), ("c", 17)], [("a", 1), ("b", 1), ("d", 1)], [("a", 2), ("c", 1), ("b", 2)],
                [("e", 16), ("a", 20)], [("e", 1), ("c", 22)], [("a", 17), ("e", 16)]]
    at = {k: 0 for k in lens}
    lines, asked = [], []
    for n, step in enumerate(schedule):
        entries, end = [], []
        for k, c in step:
            want = list(range(c))[-3:]       # the last three places of every portion
            entries.append({"id": k, "tokens": reqs[k][at[k]:at[k] + c], "want": want})
            asked += [(n, k, at[k] + w) for w in want]
            at[k] += c
            if at[k] == lens[k]:
                end.append(k)
        lines.append(json.dumps({"step": n, "entries": entries, "end": end}))
    assert at == lens
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", dtype, "--out",
                        str(out), "--max-tokens", "320"], input="\n".join(lines) + "\n", capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [f"done {n}" for n in range(len(schedule))]
    wants = {k: O.forward(f64(W), cfg, t)[0] for k, t in reqs.items()}
    got, want = [], []
    for n in range(len(schedule)):
        rows = [(k, p) for m, k, p in asked if m == n]
        got.append(torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(len(rows), cfg["vocab"])))
        want.append(torch.stack([wants[k][p] for k, p in rows]))
        if dtype == "float32":
            assert close(got[-1], want[-1], dtype), f"step {n}"
    assert close(torch.cat(got), torch.cat(want), dtype)
