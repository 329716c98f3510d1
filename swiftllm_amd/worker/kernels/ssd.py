"""A state-space recurrence with a scalar decay per head as a recurrent mixer with per-sequence state slots.
csrc/ssd.hip."""
import torch

from swiftllm_amd import _hip

from .rms_stream import StateRef


def state_space_mixer(proj: torch.Tensor, conv_w: torch.Tensor, conv_b: torch.Tensor, a_log: torch.Tensor,
                      dt_bias: torch.Tensor, d_skip: torch.Tensor, norm_w: torch.Tensor, st: StateRef, tail_off: int,
                      state_off: int, mixer, eps: float) -> torch.Tensor:
    """proj [T, z | x | B | C | dt] (rows of the input projection; a column slice of a wider matrix is fine) -> [T, heads * vdim]
    in proj's dtype: causal convolution with bias + SiLU on x | B | C (conv_w tap-major [taps, channels]), dt = softplus(dt +
    dt_bias), the token-by-token recurrence S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x on the fp32 state
    [heads, state, vdim] at `state_off` inside each sequence's slot, then y * silu(z) RMS-normed in mixer.norm_groups parts and
    scaled by norm_w."""
    _hip.require_gpu_tensor(proj, "proj")
    n = proj.shape[0]
    H, P, N, G = mixer.num_heads, mixer.value_dim, mixer.state_dim, mixer.groups
    C = mixer.conv_channels
    assert proj.stride(1) == 1 and proj.shape[1] >= mixer.proj_size
    assert conv_w.dtype == torch.float32 and conv_w.is_contiguous() and conv_w.shape == (mixer.conv_taps, C)
    for t, size in ((conv_b, C), (a_log, H), (dt_bias, H), (d_skip, H), (norm_w, mixer.inner)):
        assert t.dtype == torch.float32 and t.is_contiguous() and t.numel() == size
    dev, f32 = proj.device, torch.float32
    xbc = torch.empty((n, C), dtype=f32, device=dev)
    dt = torch.empty((n, H), dtype=f32, device=dev)
    decay = torch.empty((n, H), dtype=f32, device=dev)
    code, stream = _hip.dtype_code3(proj.dtype), _hip.stream()
    _hip.call("swl_ssd_prep", _hip.ptr(xbc), _hip.ptr(dt), _hip.ptr(decay), _hip.ptr(proj), proj.stride(0), _hip.ptr(conv_w),
              _hip.ptr(conv_b), _hip.ptr(a_log), _hip.ptr(dt_bias), _hip.ptr(st.pool), st.pool.stride(0), int(tail_off),
              _hip.ptr(st.tok_pos), _hip.ptr(st.tok_start), _hip.ptr(st.tok_state), _hip.ptr(st.tok_seq), n, H, P, N, G,
              mixer.conv_taps, code, stream)
    y = torch.empty((n, H * P), dtype=f32, device=dev)
    _hip.call("swl_ssd_scan", _hip.ptr(y), _hip.ptr(xbc), _hip.ptr(dt), _hip.ptr(decay), _hip.ptr(d_skip), _hip.ptr(st.pool),
              st.pool.stride(0), int(state_off), _hip.ptr(st.seq_row0), _hip.ptr(st.seq_cnt), _hip.ptr(st.tok_pos),
              _hip.ptr(st.tok_state), st.seq_row0.shape[0], H, P, N, G, stream)
    out = torch.empty((n, H * P), dtype=proj.dtype, device=dev)
    _hip.call("swl_gated_group_rmsnorm", _hip.ptr(out), _hip.ptr(y), _hip.ptr(proj), proj.stride(0), _hip.ptr(norm_w),
              float(eps), n, H * P, mixer.norm_groups, code, stream)
    return out
