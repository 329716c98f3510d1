#!/usr/bin/env python3
"""mixer_micro.py --kernel ssd|sigmoid [--tokens N --seqs S --heads H --dim D --iters K] — launches of one mixer kernel at a
prompt's shape (S portions of N tokens) or a decode step's (N = 1 at context --context), timed with HIP events; one JSON line.
Under `rocprofv3 --pmc ... --kernel-trace` it is the program whose counters tools/rocpd_pmc.py summarises."""
import argparse
import json
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def i32(xs):
    return torch.tensor(xs, dtype=torch.int32, device="cuda")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--kernel", required=True, choices=["ssd", "sigmoid"])
    ap.add_argument("--tokens", type=int, default=2048)
    ap.add_argument("--seqs", type=int, default=4)
    ap.add_argument("--context", type=int, default=0, help="tokens already cached per sequence")
    ap.add_argument("--heads", type=int, default=8)
    ap.add_argument("--kv-heads", type=int, default=2)
    ap.add_argument("--dim", type=int, default=128)
    ap.add_argument("--iters", type=int, default=12)
    a = ap.parse_args()
    from swiftllm_amd import _hip
    from swiftllm_amd.model_config import RatilornAttentionConfig, StateSpaceConfig
    from swiftllm_amd.worker.kernels.rms_stream import StateRef
    _hip.load()
    S, N, H, d, ctx = a.seqs, a.tokens, a.heads, a.dim, a.context
    T = S * N
    seq = [s for s in range(S) for _ in range(N)]
    pos = [ctx + j for _ in range(S) for j in range(N)]
    g = torch.Generator(device="cuda").manual_seed(0)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    if a.kernel == "ssd":
        from swiftllm_amd.worker.kernels.ssd import state_space_mixer
        mx = StateSpaceConfig(dict(heads=H, vdim=d, state=d, groups=1, conv=4, norm_groups=1))
        slot = 2 * 3 * mx.conv_channels + mx.state_elems
        pool = torch.zeros((S, slot), dtype=torch.float32, device="cuda")
        st = StateRef(pool, i32(pos), i32([ctx] * T), i32([2 * s for s in seq]), i32(seq), i32([s * N for s in range(S)]),
                      i32([N] * S))
        proj = (torch.randn((T, mx.proj_size + 8), generator=g, device="cuda") * 0.5).to(torch.bfloat16)
        f = lambda *shape: torch.randn(shape, generator=g, device="cuda") * 0.3
        args = (proj, f(4, mx.conv_channels), f(mx.conv_channels), f(H), f(H), f(H), 1 + f(mx.inner), st, 0,
                2 * 3 * mx.conv_channels, mx, 1e-6)
        run = lambda: state_space_mixer(*args)
        what = dict(kernel="ssd_prep + ssd_scan + gated_group_rmsnorm", state=[H, d, d])
    else:
        from swiftllm_amd.worker.kernels.sigmoid_attn import sigmoid_attention
        from swiftllm_amd.worker.kernels.window_attn import PoolSlice
        mx = RatilornAttentionConfig(dict(heads=H, kv_heads=a.kv_heads, dim=d, vdim=d, scale=d ** -0.5), True)
        per = -(-(ctx + N) // 16)
        table = torch.randperm(S * per, generator=torch.Generator().manual_seed(1)).to(torch.int32).view(S, per).cuda()
        pool = (torch.randn((S * per, (mx.k_size + mx.v_size) * 16), generator=g, device="cuda")).to(torch.bfloat16)
        q = torch.randn((T, mx.q_size), generator=g, device="cuda").to(torch.bfloat16)
        row0 = [s * N + t for s in range(S) for t in range(0, N, 16)]
        cnt = [min(16, N - t) for s in range(S) for t in range(0, N, 16)]
        f = lambda *shape: torch.rand(shape, generator=g, device="cuda")
        talk = (torch.eye(H, device="cuda") + 0.1 * f(H, H)).contiguous()
        args = (q, pool, PoolSlice(0, mx.k_size * 16), table, i32(seq), i32(pos), mx, talk, f(H), f(H), -2 + f(H),
                (i32(row0), i32(cnt)), ctx + N)
        run = lambda: sigmoid_attention(*args)
        what = dict(kernel="sigmoid_attn_mfma (+ sum of the key shares)", heads=[H, a.kv_heads, d])
    run()
    torch.cuda.synchronize()
    ev[0].record()
    for _ in range(a.iters):
        run()
    ev[1].record()
    torch.cuda.synchronize()
    print(json.dumps(dict(what, seqs=S, tokens=N, context=ctx, us_per_call=ev[0].elapsed_time(ev[1]) * 1e3 / a.iters)))


if __name__ == "__main__":
    main()
