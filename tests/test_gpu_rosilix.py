"""Rosilix on the GPU against the plain implementation in tests/rosilix_oracle.py: every mechanism alone, whole prompts,
token-by-token decoding, portions down to two tokens, unequal batches, reused blocks and block-table rows, far keys, keys at
page borders and at both sides of a chunk's edge, the first tokens of a sequence, long decoding, odd sizes, hipGraph replays,
swapping, and greedy generation through the Engine and its scheduler. Configurations and weights are made here (small,
random, seeded)."""
import asyncio
import json
import os

import pytest
import torch

import rosilix_oracle as O

pytestmark = pytest.mark.gpu

F32_TOL = 3e-5      # relative rms error of fp32 logits (true fp32 products, fp32 statistics)
BF16_TOL = 8e-2     # the same in bfloat16 (bf16 products and activations, fp32 stream, scores and statistics)


def write_model(path, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


def make_model(path, cfg, W, dtype="float32", num_blocks=48, max_seqs=4, cpu_blocks=0, graph=False, max_len=512):
    from swiftllm_amd import EngineConfig, build_model
    write_model(path, cfg, W)
    ecfg = EngineConfig(model_path=str(path), use_dummy=False, block_size=16, gpu_mem_utilization=0.9,
                        num_cpu_blocks=cpu_blocks, max_seqs_in_block_table=max_seqs, max_blocks_per_seq=-(-max_len // 16),
                        max_batch_size=max_seqs, max_tokens_in_batch=1024, dtype=dtype, use_hip_graph=graph)
    model = build_model(ecfg)
    model.load_weights()
    model.init_kvcache_and_swap(num_blocks)
    return model


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-9)).max())


def close(got, want, dtype, tol):
    """fp32: every position within the tolerance. bfloat16: rounding is amplified where a unit-RMS norm meets a small vector,
    so 19 of 20 positions are held to the tolerance and every position to three times it."""
    if dtype == "float32":
        return rel_err(got, want) < tol
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-9)
    return float(e.max()) < 3 * tol and float((e < tol).double().mean()) >= 0.95


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


# ---- mechanisms alone --------------------------------------------------------------------------------------------------------
class MixerBench:
    """One mixer of the product on a hand-made pool: its weights loaded by the product's loader from a dict, a block table
    in which another sequence owns the first blocks, a pool full of finite garbage."""

    def __init__(self, layers, W, dtype, which=0, width=64, num_blocks=40):
        from swiftllm_amd.model_config import RosilixModelConfig
        from swiftllm_amd.worker.block_manager import BlockManager
        from swiftllm_amd.worker.kernels.window_attn import PoolSlice
        from swiftllm_amd.worker.layers.rosilix_layer import RosilixDiffAttention, RosilixLatentAttention
        from swiftllm_amd.worker.rosilix_weight import RosilixLayerWeight
        self.cfg = RosilixModelConfig(O.make_config(layers, width=width))
        self.dtype = dtype

        def get(name, shape):
            t = W[name]
            assert tuple(t.shape) == tuple(shape), name
            return t
        self.mgr = BlockManager("GPU", num_blocks, 3, num_blocks, 16, "cuda")
        self.mgr.allocate_blocks_for_seqs([1], [37])         # another sequence owns the first blocks
        self.ops, off = [], 24
        slices = {}
        for i, lcfg in enumerate(self.cfg.layers):
            lw = RosilixLayerWeight(i)
            lw.load(get, self.cfg, lcfg, dtype, torch.device("cuda"))
            if lcfg.mixer.kv_from < 0:
                slices[i] = PoolSlice(off, off + lcfg.mixer.k_size * 16)
                off += (lcfg.mixer.k_size + lcfg.mixer.v_size) * 16 + 8
            else:
                slices[i] = slices[lcfg.mixer.kv_from]
            kind = RosilixDiffAttention if lcfg.type == "attention" else RosilixLatentAttention
            self.ops.append(kind(lcfg, lw, self.cfg.norm_eps, False, slices[i], 512))
        self.pool = torch.full((num_blocks, off + 16), 3e4, dtype=dtype, device="cuda")
        self.which = which

    def run(self, hs, portions, tiled, seq=2):
        """hs: one input [n, width] per layer of the bench (a borrowing layer needs its lender to have run on the same
        tokens); -> output of layer `which`, portions concatenated."""
        from swiftllm_amd.worker.layers.lorulix_layer import StepContext
        n = hs[0].shape[0]
        out, at = [], 0
        for c in list(portions) * n:
            if at >= n:
                break
            c = min(c, n - at)
            self.mgr.allocate_blocks_for_seqs([seq], [at + c])
            pos = torch.arange(at, at + c, dtype=torch.int32, device="cuda")
            sq = torch.full((c,), seq, dtype=torch.int32, device="cuda")
            tiles = None
            if tiled:
                r0 = torch.arange(0, c, 16, dtype=torch.int32)
                tiles = (r0.cuda(), torch.minimum(torch.full_like(r0, 16), c - r0).cuda())
            ctx = StepContext(self.pool, self.mgr.block_table, sq, pos, tiles, None)
            for i, op in enumerate(self.ops):
                y = op.forward(hs[i][at:at + c].to(self.dtype).cuda(), ctx)
                if i == self.which:
                    out.append(y.cpu())
            at += c
        return torch.cat(out).double()


def layer_weights(layers, seed, width=64):
    cfg = O.make_config(layers, width=width)
    return cfg, O.make_weights(cfg, seed=seed, dtype=torch.float32)


def mixer_tol(dtype, want):
    return (2e-4 if dtype == torch.float32 else 4e-2) * max(1.0, float(want.abs().max()))


@pytest.mark.parametrize("H,G,d,e,chunk,rot,n", [(4, 2, 16, 24, 24, 8, 150), (3, 1, 10, 6, 7, 10, 70), (2, 2, 8, 8, None, 2, 33),
                                                 (5, 5, 12, 20, 16, 0, 50), (1, 1, 32, 16, 100, 32, 1),
                                                 (20, 4, 8, 12, 30, 4, 40), (6, 2, 64, 320, 20, 16, 35)])
def test_differential_attention_alone(H, G, d, e, chunk, rot, n):
    """The mixer in fp32 (the plain kernels), whole and in portions that cut chunks and pages anywhere."""
    layers = [O.diff_mixer(heads=H, kv_heads=G, dim=d, vdim=e, chunk=chunk, rot_dims=rot, diff=0.35, scale=0.4)]
    cfg, W = layer_weights(layers, seed=n + H)
    g = torch.Generator().manual_seed(n)
    h = torch.randn(n, 64, generator=g)
    want = O.diff_attention_mixer(h.double(), {k: v.double() for k, v in W.items()}, "l0.mix.", cfg["layers"][0]["mixer"], 1e-5)
    for portions in ((1000,), (5, 1, 2, 30), (1,)):
        got = MixerBench(layers, W, torch.float32).run([h], portions, False)
        assert (got - want).abs().max() < mixer_tol(torch.float32, want), portions


@pytest.mark.parametrize("H,G,d,e,chunk,n", [(4, 1, 64, 128, 48, 150), (2, 2, 48, 96, 40, 90), (8, 2, 32, 64, None, 70),
                                             (16, 4, 64, 64, 64, 64), (3, 1, 128, 128, 33, 80)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_differential_attention_on_the_matrix_cores(H, G, d, e, chunk, n, dtype):
    layers = [O.diff_mixer(heads=H, kv_heads=G, dim=d, vdim=e, chunk=chunk, rot_dims=d // 2, diff=0.2, scale=d ** -0.5)]
    cfg, W = layer_weights(layers, seed=n, width=128)
    W = {k: v.to(dtype).float() for k, v in W.items()}
    g = torch.Generator().manual_seed(n)
    h = torch.randn(n, 128, generator=g).to(dtype).float()
    want = O.diff_attention_mixer(h.double(), {k: v.double() for k, v in W.items()}, "l0.mix.", cfg["layers"][0]["mixer"], 1e-5)
    tiled = MixerBench(layers, W, dtype, width=128).run([h], (17, 1, 2, 40), True)
    plain = MixerBench(layers, W, dtype, width=128).run([h], (17, 1, 2, 40), False)
    assert (tiled - want).abs().max() < mixer_tol(dtype, want)
    assert (plain - want).abs().max() < mixer_tol(dtype, want)


@pytest.mark.parametrize("H,d,dr,e,r,n", [(3, 16, 8, 24, 32, 150), (5, 8, 4, 8, 12, 70), (1, 24, 16, 40, 20, 33),
                                          (6, 4, 2, 6, 7, 45), (2, 16, 16, 16, 16, 1)])
def test_latent_attention_alone_and_borrowed(H, d, dr, e, r, n):
    """fp32: a latent layer and a second one (other head count and sizes) that reads the first one's cache."""
    layers = [O.latent_mixer(heads=H, dim=d, rot_dim=dr, vdim=e, kv_rank=r, base=300.0, scale=0.3),
              O.latent_mixer(heads=H + 1, dim=d + 2, rot_dim=dr, vdim=e + 4, kv_rank=r, base=300.0, kv_from=0, scale=0.2)]
    cfg, W = layer_weights(layers, seed=n + H)
    W64 = {k: v.double() for k, v in W.items()}
    g = torch.Generator().manual_seed(n)
    h0, h1 = torch.randn(n, 64, generator=g), torch.randn(n, 64, generator=g)
    mx0, mx1 = cfg["layers"][0]["mixer"], cfg["layers"][1]["mixer"]
    kv = O.latent_kv(h0.double(), W64, "l0.mix.", mx0, 1e-5)
    want0 = O.latent_attention_mixer(h0.double(), W64, "l0.mix.", mx0, 1e-5, kv)
    want1 = O.latent_attention_mixer(h1.double(), W64, "l1.mix.", mx1, 1e-5, kv)
    for portions in ((1000,), (5, 1, 2, 30), (1,)):
        assert (MixerBench(layers, W, torch.float32, 0).run([h0, h1], portions, False) - want0).abs().max() < \
            mixer_tol(torch.float32, want0), portions
        assert (MixerBench(layers, W, torch.float32, 1).run([h0, h1], portions, False) - want1).abs().max() < \
            mixer_tol(torch.float32, want1), portions


@pytest.mark.parametrize("H,d,dr,e,r,n", [(6, 32, 32, 48, 64, 150), (4, 64, 32, 64, 96, 90), (16, 16, 16, 32, 48, 70),
                                          (40, 8, 32, 16, 32, 40), (2, 64, 64, 128, 128, 50), (6, 32, 64, 32, 512, 60),
                                          (3, 16, 32, 48, 256, 45)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_latent_attention_on_the_matrix_cores(H, d, dr, e, r, n, dtype):
    layers = [O.latent_mixer(heads=H, dim=d, rot_dim=dr, vdim=e, kv_rank=r, scale=(d + dr) ** -0.5)]
    cfg, W = layer_weights(layers, seed=n, width=128)
    W = {k: v.to(dtype).float() for k, v in W.items()}
    W64 = {k: v.double() for k, v in W.items()}
    g = torch.Generator().manual_seed(n)
    h = torch.randn(n, 128, generator=g).to(dtype).float()
    mx = cfg["layers"][0]["mixer"]
    want = O.latent_attention_mixer(h.double(), W64, "l0.mix.", mx, 1e-5, O.latent_kv(h.double(), W64, "l0.mix.", mx, 1e-5))
    tiled = MixerBench(layers, W, dtype, width=128).run([h], (17, 1, 2, 40), True)
    assert (tiled - want).abs().max() < mixer_tol(dtype, want)
    plain = MixerBench(layers, W, dtype, width=128).run([h], (17, 1, 2, 40), False)
    assert (plain - want).abs().max() < mixer_tol(dtype, want)


def test_the_sink_takes_its_share():
    """Sinks far above and far below the scores: nearly all weight goes to the sink (the output vanishes), or none."""
    layers = [O.latent_mixer(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=32, scale=0.1)]
    cfg, W = layer_weights(layers, seed=1)
    g = torch.Generator().manual_seed(2)
    h = torch.randn(40, 64, generator=g)
    mx = cfg["layers"][0]["mixer"]
    for tiled, dtype in ((False, torch.float32), (True, torch.bfloat16)):
        for sinks in ([30.0, -30.0], [-60.0, 90.0], [0.0, 3.0]):
            W["l0.mix.sink"] = torch.tensor(sinks)
            W64 = {k: v.to(dtype).double() for k, v in W.items()}
            hh = h.to(dtype).double()
            want = O.latent_attention_mixer(hh, W64, "l0.mix.", mx, 1e-5, O.latent_kv(hh, W64, "l0.mix.", mx, 1e-5))
            got = MixerBench(layers, {k: v.to(dtype).float() for k, v in W.items()}, dtype).run([h], (13, 1, 2), tiled)
            assert (got - want).abs().max() < mixer_tol(dtype, want), (tiled, sinks)


def _aligned_diff_case(chunk, n, target, d=16, e=16, scale=1.0):
    """A differential layer whose first score map's queries equal its keys, and inputs in which the tokens from `target` on
    share one strong direction with token `target`: the key at `target` then dominates map 1 of every later query that may
    see it, and a key that is wrongly seen or wrongly hidden moves the output by far more than rounding."""
    layers = [O.diff_mixer(heads=2, kv_heads=1, dim=d, vdim=e, chunk=chunk, rot_dims=4, diff=0.3, scale=scale)]
    cfg, W = layer_weights(layers, seed=7)
    q = W["l0.mix.q"].view(2, 2, d, 64)
    k = W["l0.mix.k"].view(1, 2, d, 64)
    q[:, 0] = k[0, 0]
    W["l0.mix.q"] = q.reshape(-1, 64).contiguous()
    g = torch.Generator().manual_seed(n)
    h = 0.05 * torch.randn(n, 64, generator=g)
    u = torch.randn(64, generator=g)
    h[target] += 1.5 * u
    h[target + 1:] += 1.5 * u * (torch.arange(n - target - 1) % 2 == 0).float()[:, None]     # every second later token asks
    return layers, cfg, W, h


@pytest.mark.parametrize("tiled,dtype", [(False, torch.float32), (True, torch.bfloat16)])
@pytest.mark.parametrize("chunk,n,target", [(None, 400, 3), (None, 400, 15), (None, 400, 16), (48, 150, 96), (48, 150, 95),
                                            (48, 150, 47), (40, 130, 80), (40, 130, 79)])
def test_keys_far_away_at_page_borders_and_at_chunk_edges(tiled, dtype, chunk, n, target):
    """The dominant key hundreds of positions back, on both sides of a page border, as the first key of a chunk (every query
    of the chunk sees it) and as the last key of the chunk before (no later query may): in prompt portions and decoded."""
    # (16-bit runs: the dominant score is kept near 14, so that the rounding of queries and keys does not move the weights)
    layers, cfg, W, h = _aligned_diff_case(chunk, n, target, d=16 if not tiled else 32, e=16 if not tiled else 32,
                                           scale=1.0 if dtype == torch.float32 else 0.05)
    Wd = {k: v.to(dtype).float() for k, v in W.items()}
    hd = h.to(dtype).float()
    want = O.diff_attention_mixer(hd.double(), {k: v.double() for k, v in Wd.items()}, "l0.mix.", cfg["layers"][0]["mixer"], 1e-5)
    for portions in ((n - 30, 1), (37, 2, 1, 16)):
        got = MixerBench(layers, Wd, dtype).run([hd], portions, tiled)
        assert (got - want).abs().max() < mixer_tol(dtype, want), portions
    if chunk:   # the case is sharp: hiding the first key of the chunk, or showing the last of the one before, would show
        mx = dict(cfg["layers"][0]["mixer"], mask={"size": chunk + 1})
        other = O.diff_attention_mixer(hd.double(), {k: v.double() for k, v in Wd.items()}, "l0.mix.", mx, 1e-5)
        assert (other - want).abs().max() > 20 * mixer_tol(dtype, want)


@pytest.mark.parametrize("tiled,dtype", [(False, torch.float32), (True, torch.bfloat16)])
def test_a_far_latent_key_among_hundreds_is_found(tiled, dtype):
    """The key up-projection gets a rank-one term that turns the latent of one early token into the direction the late
    queries ask for; every other key is noise."""
    n, target, H, d, dr, r = 420, 5, 2, 32, 32, 32
    gain = 124.0        # (the target's score: scale * gain * sqrt(r) = 14; the other keys' scores have a deviation below 1)
    layers = [O.latent_mixer(heads=H, dim=d, rot_dim=dr, vdim=32, kv_rank=r, scale=0.02)]
    cfg, W = layer_weights(layers, seed=11)
    mx = cfg["layers"][0]["mixer"]
    g = torch.Generator().manual_seed(4)
    h = 0.3 * torch.randn(n, 64, generator=g)
    u = torch.randn(64, generator=g)
    h[-40:] = u + 0.05 * torch.randn(40, 64, generator=g)
    W["l0.mix.sink"] = torch.zeros(H)
    c, _ = O.latent_kv(h.double(), {k: v.double() for k, v in W.items()}, "l0.mix.", mx, 1e-5)
    cj = c[target].float()
    qu = (W["l0.mix.q"] @ u).view(H, d + dr)[:, :d]
    uk = W["l0.mix.uk"].view(H, d, r)
    for hd in range(H):
        uk[hd] += gain * torch.outer(qu[hd] / qu[hd].norm() ** 2, cj / cj.norm() ** 2 * r ** 0.5)
    W["l0.mix.uk"] = uk.reshape(H * d, r).contiguous()
    Wd = {k: v.to(dtype).float() for k, v in W.items()}
    hd_ = h.to(dtype).float()
    W64 = {k: v.double() for k, v in Wd.items()}
    kv = O.latent_kv(hd_.double(), W64, "l0.mix.", mx, 1e-5)
    want = O.latent_attention_mixer(hd_.double(), W64, "l0.mix.", mx, 1e-5, kv)
    for portions in ((n - 30, 1), (97, 2, 1, 16)):
        got = MixerBench(layers, Wd, dtype).run([hd_], portions, tiled)
        assert (got - want).abs().max() < mixer_tol(dtype, want), portions
    # sharp: without the target key the late outputs are different
    hidden = torch.cat((hd_[:target], hd_[target + 1:]))
    kv2 = O.latent_kv(hidden.double(), W64, "l0.mix.", mx, 1e-5)
    other = O.latent_attention_mixer(hidden.double(), W64, "l0.mix.", mx, 1e-5, kv2)
    assert (other[-20:] - want[-20:]).abs().max() > 5 * mixer_tol(dtype, want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotation_and_store_kernel(dtype):
    """Rows [q | k | v | extra columns]: queries rotated in place, keys rotated into the pages, values transposed into them,
    at positions up to 100000 (angles in float64)."""
    from swiftllm_amd.worker.block_manager import BlockManager
    from swiftllm_amd.worker.kernels.rope_kv import rope_and_store_kv
    from swiftllm_amd.worker.kernels.window_attn import PoolSlice
    nq, nk, nv, d, dv, rot, base = 5, 3, 2, 12, 10, 8, 777.0
    g = torch.Generator().manual_seed(0)
    n = 21
    rows = torch.randn(n, (nq + nk) * d + nv * dv + 5, generator=g).to(dtype)
    start = 99990
    mgr = BlockManager("GPU", 7000, 2, 6300, 16, "cuda")
    mgr.allocate_blocks_for_seqs([1], [start + n])
    pos = torch.arange(start, start + n, dtype=torch.int32)
    freq = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float64).cuda()
    sl = PoolSlice(8, 8 + nk * d * 16)
    pool = torch.zeros((7000, 8 + (nk * d + nv * dv) * 16), dtype=dtype, device="cuda")
    dev = rows.cuda()
    rope_and_store_kv(dev, freq, rot, pool, sl, mgr.block_table, torch.ones(n, dtype=torch.int32).cuda(), pos.cuda(),
                      nq, nk, nv, d, dv)
    r64 = rows.double()
    qk = O.rotate_pairs(r64[:, :(nq + nk) * d].reshape(n, nq + nk, d), pos, rot, base)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert (dev.cpu().double()[:, :nq * d] - qk[:, :nq].reshape(n, -1)).abs().max() < tol
    assert torch.equal(dev.cpu()[:, nq * d:], rows[:, nq * d:])            # everything after the queries is untouched
    table = mgr.block_table[1].cpu()
    for t in range(n):
        page = pool[int(table[(start + t) // 16])].cpu().double()
        o = (start + t) % 16
        kk = page[8:8 + nk * d * 16].view(nk, 16, d)[:, o]
        vv = page[8 + nk * d * 16:].view(nv, dv, 16)[:, :, o]
        assert (kk - qk[t, nq:]).abs().max() < tol
        assert torch.equal(vv.reshape(-1), r64[t, (nq + nk) * d:(nq + nk) * d + nv * dv])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_map_combination_and_head_gate(dtype):
    from swiftllm_amd.worker.kernels.rope_kv import diff_head_combine, head_gate_
    g = torch.Generator().manual_seed(1)
    n, H, e, lam, mult, eps = 19, 5, 24, 0.37, 0.7, 1e-5
    maps = torch.randn(n, 2, H, e, generator=g)
    wide = torch.randn(n, H + 3, generator=g).to(dtype)
    gate = wide[:, 2:2 + H]
    o = maps[:, 0].double() - lam * maps[:, 1].double()
    want = O.unit_rms(o, eps) * mult * torch.sigmoid(gate.double())[:, :, None]
    got = diff_head_combine(maps.view(n, -1).cuda(), wide.cuda()[:, 2:2 + H], lam, mult, eps, H, e, dtype)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert (got.cpu().double().view(n, H, e) - want).abs().max() < tol
    y = torch.randn(n, H * e, generator=g).to(dtype)
    got = head_gate_(y.cuda().clone(), wide.cuda()[:, 2:2 + H], H, e)
    assert (got.cpu().double().view(n, H, e) - y.double().view(n, H, e) * torch.sigmoid(gate.double())[:, :, None]).abs().max() < tol


def test_embedding_without_positions_and_squared_relu():
    from swiftllm_amd.worker.kernels.layernorm import embed_positions
    from swiftllm_amd.worker.kernels.moe import relu_squared
    g = torch.Generator().manual_seed(2)
    emb = torch.randn(30, 40, generator=g).to(torch.bfloat16)
    ids = torch.tensor([3, 29, 0, 3], dtype=torch.int32)
    x, _ = embed_positions(ids.cuda(), None, emb.cuda(), None, 2.5, keep_copy=False)
    assert torch.equal(x.cpu(), emb[ids.long()].float() * 2.5)
    z = torch.randn(7, 33, generator=g)
    assert torch.allclose(relu_squared(z.cuda(), 33).cpu(), torch.relu(z) ** 2)


# ---- the whole model -------------------------------------------------------------------------------------------------------
def default_layers():
    return [O.latent_mixer(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=32),
            O.diff_mixer(heads=4, kv_heads=2, dim=16, vdim=32, chunk=24, rot_dims=8),
            O.latent_mixer(heads=2, dim=8, rot_dim=8, vdim=16, kv_rank=32, kv_from=0),
            O.diff_mixer(heads=2, kv_heads=1, dim=8, vdim=8, chunk=10, rot_dims=8, diff=0.4)]


@pytest.fixture(scope="module")
def default_case():
    cfg = O.make_config(default_layers(), no_mlp=(2,))
    W = O.make_weights(cfg, seed=3)
    toks = tokens_for(cfg, 90, 1)
    streams = []
    logits = O.forward(cfg, W, toks, streams)
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
    want_other = O.forward(cfg, W, other)
    a = [model.step([entry(0, toks[:30], 0), entry(1, other[:11], 0)])]
    got0, got1 = [a[0][:30]], [a[0][30:]]
    for i in range(40):     # two sequences decode together: one captured graph, replayed with other positions and pages
        lg = model.step([entry(0, toks[30 + i:31 + i], 30 + i), entry(1, other[11 + i:12 + i], 11 + i)]).clone()
        got0.append(lg[:1])
        got1.append(lg[1:])
        torch.cuda.synchronize()
    assert model.graph_captures == 1
    assert rel_err(torch.cat(got0), want[:70]) < F32_TOL
    assert rel_err(torch.cat(got1), want_other[:51]) < F32_TOL


@pytest.mark.parametrize("dtype,tol", [("float32", F32_TOL), ("bfloat16", BF16_TOL)])
def test_unequal_batches_and_reused_blocks(tmp_path, default_case, dtype, tol):
    """Four live requests of unequal length, portions beside decoded tokens; finished requests give their blocks and block
    table rows to new ones. Every request's logits equal those of the request alone."""
    cfg, W, _, _, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, dtype, num_blocks=20, max_seqs=4)
    lens = [70, 5, 33, 1, 48, 17, 2]
    reqs = [tokens_for(cfg, n, 50 + i) for i, n in enumerate(lens)]
    wants = [O.forward(cfg, W, t) for t in reqs]
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
    assert model.gpu_block_manager.num_free_blocks == 20
    for r in range(len(reqs)):
        assert close(torch.cat(got[r]), wants[r], dtype, tol), f"request {r}"


def varied_layers():
    """Sizes that a symmetric configuration would hide: dim != vdim, heads not a power of two, one kv head and heads = kv
    heads, a rotation of the whole head and of a part of it, no chunks, chunks of one page and chunks that are no multiple of
    a page, a differential layer first, two layers that read the same latent cache, a latent size below the head size."""
    return [O.diff_mixer(heads=3, kv_heads=3, dim=24, vdim=8, chunk=None, rot_dims=24, diff=0.1),
            O.latent_mixer(heads=5, dim=8, rot_dim=4, vdim=40, kv_rank=6, base=50.0),
            O.diff_mixer(heads=6, kv_heads=1, dim=8, vdim=24, chunk=16, rot_dims=2, diff=0.6),
            O.latent_mixer(heads=1, dim=24, rot_dim=4, vdim=8, kv_rank=6, base=50.0, kv_from=1),
            O.latent_mixer(heads=4, dim=8, rot_dim=4, vdim=8, kv_rank=6, base=50.0, kv_from=1),
            O.diff_mixer(heads=2, kv_heads=2, dim=16, vdim=16, chunk=37, rot_dims=8, diff=0.5),
            O.latent_mixer(heads=2, dim=16, rot_dim=16, vdim=16, kv_rank=48)]


@pytest.mark.parametrize("dtype,tol", [("float32", F32_TOL), ("bfloat16", BF16_TOL)])
def test_other_sizes(tmp_path, dtype, tol):
    cfg = O.make_config(varied_layers(), width=48, vocab=75, ff=56, embed_scale=1.0, no_mlp=(0, 4))
    W = O.make_weights(cfg, seed=4)
    toks = tokens_for(cfg, 120, 5)
    want = O.forward(cfg, W, toks)
    model = make_model(tmp_path / "m", cfg, W, dtype)
    assert close(model.step([entry(0, toks, 0)]), want, dtype, tol)
    assert close(run_in_portions(model, 1, toks, [7, 1, 2, 33, 1]), want, dtype, tol)
    assert close(run_in_portions(model, 2, toks, [100, 1]), want, dtype, tol)


@pytest.mark.parametrize("dtype,tol", [("float32", F32_TOL), ("bfloat16", BF16_TOL)])
def test_sizes_that_are_multiples_of_two_only(tmp_path, dtype, tol):
    """Width, vocabulary, feed-forward, head and latent sizes that are multiples of nothing but 2: no kernel or projection may
    lean on an alignment that the common sizes happen to have. Chunks of one position: a token sees itself only."""
    layers = [O.latent_mixer(heads=3, dim=6, rot_dim=10, vdim=14, kv_rank=22, base=33.0),
              O.diff_mixer(heads=3, kv_heads=1, dim=10, vdim=6, chunk=13, rot_dims=6, diff=0.2),
              O.diff_mixer(heads=2, kv_heads=2, dim=6, vdim=22, chunk=1, rot_dims=6, diff=0.45),
              O.latent_mixer(heads=7, dim=10, rot_dim=10, vdim=6, kv_rank=22, base=33.0, kv_from=0)]
    cfg = O.make_config(layers, width=50, vocab=77, ff=54, embed_scale=7.0, no_mlp=(1,))
    W = O.make_weights(cfg, seed=9)
    toks = tokens_for(cfg, 75, 9)
    want = O.forward(cfg, W, toks)
    model = make_model(tmp_path / "m", cfg, W, dtype)
    assert close(model.step([entry(0, toks, 0)]), want, dtype, tol)
    assert close(run_in_portions(model, 1, toks, [3, 1, 2, 29, 1]), want, dtype, tol)


def test_matrix_core_paths_in_the_model(tmp_path):
    """bfloat16 with head sizes the tiled attention serves: a prompt in portions and decoded tokens against the oracle on the
    same (bf16-representable) weights, with the packed decode projections."""
    layers = [O.latent_mixer(heads=8, dim=32, rot_dim=32, vdim=32, kv_rank=64),
              O.diff_mixer(heads=4, kv_heads=2, dim=64, vdim=128, chunk=48, rot_dims=32),
              O.latent_mixer(heads=4, dim=64, rot_dim=32, vdim=64, kv_rank=64, kv_from=0),
              O.diff_mixer(heads=4, kv_heads=1, dim=32, vdim=64, chunk=None, rot_dims=32)]
    cfg = O.make_config(layers, width=128, vocab=160, ff=256)
    W = O.make_weights(cfg, seed=5)
    toks = tokens_for(cfg, 140, 6)
    want = O.forward(cfg, W, toks)
    model = make_model(tmp_path / "m", cfg, W, "bfloat16")
    assert close(model.step([entry(0, toks, 0)]), want, "bfloat16", BF16_TOL)
    assert close(run_in_portions(model, 1, toks, [33, 2, 64, 1]), want, "bfloat16", BF16_TOL)


def test_decoding_batches_with_heads_on_the_tile_rows(tmp_path):
    """bfloat16 decode steps of several sequences of unequal length: every tile is one token, and the latent layers (20 and 6
    heads over one cached row: a full group of sixteen heads and a partial one) run with their heads on the matrix-core
    tile's rows; with hipGraph replay."""
    layers = [O.latent_mixer(heads=20, dim=16, rot_dim=32, vdim=16, kv_rank=64),
              O.diff_mixer(heads=2, kv_heads=1, dim=32, vdim=64, chunk=32, rot_dims=16),
              O.latent_mixer(heads=6, dim=32, rot_dim=32, vdim=48, kv_rank=64, kv_from=0)]
    cfg = O.make_config(layers, width=128, vocab=160, ff=128)
    W = O.make_weights(cfg, seed=12)
    lens, starts = [150, 61, 97], [100, 3, 48]
    reqs = [tokens_for(cfg, n, 70 + i) for i, n in enumerate(lens)]
    wants = [O.forward(cfg, W, t) for t in reqs]
    model = make_model(tmp_path / "m", cfg, W, "bfloat16", graph=True)
    got = [[model.step([entry(i, reqs[i][:starts[i]], 0)])] for i in range(3)]
    at = list(starts)
    while any(a < n for a, n in zip(at, lens)):
        live = [i for i in range(3) if at[i] < lens[i]]
        lg = model.step([entry(i, reqs[i][at[i]:at[i] + 1], at[i]) for i in live]).clone()
        for k, i in enumerate(live):
            got[i].append(lg[k:k + 1])
            at[i] += 1
    for i in range(3):
        assert close(torch.cat(got[i]), wants[i], "bfloat16", BF16_TOL), f"request {i}"


def test_first_tokens_of_a_sequence(tmp_path, default_case):
    """Sequences of one to four tokens, alone and decoded, in blocks that longer sequences used before."""
    cfg, W, toks, want, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, "float32", max_seqs=2)
    model.step([entry(0, toks, 0, want=[]), entry(1, toks[::-1], 0, want=[])])
    model.free_seqs_resources([0, 1])
    for n in (1, 2, 3, 4):
        assert rel_err(model.step([entry(0, toks[:n], 0)]), want[:n]) < F32_TOL
        assert rel_err(run_in_portions(model, 1, toks[:n], [1]), want[:n]) < F32_TOL
        model.free_seqs_resources([0, 1])


def test_long_decoding(tmp_path):
    cfg = O.make_config(default_layers())
    W = O.make_weights(cfg, seed=8)
    toks = tokens_for(cfg, 330, 3)
    want = O.forward(cfg, W, toks)
    model = make_model(tmp_path / "m", cfg, W, "float32", num_blocks=24)
    assert rel_err(run_in_portions(model, 0, toks, [10, 1]), want) < F32_TOL


def test_swap_out_and_in_keeps_the_sequence(tmp_path, default_case):
    cfg, W, toks, want, _ = default_case
    model = make_model(tmp_path / "m", cfg, W, "float32", num_blocks=12, cpu_blocks=8, max_seqs=2)
    first = model.step([entry(0, toks[:40], 0)])
    model.swap_out_seqs([0])
    assert model.gpu_block_manager.num_free_blocks == 12
    model.step([entry(1, tokens_for(cfg, 100, 1), 0, want=[])])      # overwrites the freed blocks
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
            lg = O.forward(cfg, W, seq)[-1]
            top2 = torch.topk(lg, 2).values
            assert float(top2[0] - top2[1]) > 1e-4, "the test's weights make a close call"
            seq.append(int(torch.argmax(lg)))
        return seq[len(prompt):]

    async def run():
        engine = Engine(ecfg)
        await engine.initialize()
        assert type(engine.model).__name__ == "RosilixModel"
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


@pytest.mark.parametrize("dtype,tol", [("float32", F32_TOL), ("bfloat16", BF16_TOL)])
def test_trace_runner_replays_a_mixed_schedule(tmp_path, dtype, tol):
    """bin/trace_run as a user starts it: five requests through four block-table rows and a pool of 20 blocks, portions
    beside decoded tokens, a request that sits steps out, finished requests whose blocks the next one takes."""
    import subprocess
    import sys
    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = O.make_config(default_layers(), no_mlp=(2,))
    W = O.make_weights(cfg, seed=13)
    path = write_model(tmp_path / "m", cfg, W)
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
    wants = {k: O.forward(cfg, W, t) for k, t in reqs.items()}
    got, want = [], []
    for n in range(len(schedule)):
        rows = [(k, p) for m, k, p in asked if m == n]
        got.append(torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(len(rows), cfg["vocab"])))
        want.append(torch.stack([wants[k][p] for k, p in rows]))
        if dtype == "float32":
            assert close(got[-1], want[-1], dtype, tol), f"step {n}"
    assert close(torch.cat(got), torch.cat(want), dtype, tol)

