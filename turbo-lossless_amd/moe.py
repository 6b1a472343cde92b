"""Mixture-of-experts SwiGLU FFN over split-12 experts: tokens grouped per expert, each group
through the fused decode+GEMM (w1|w3 as one two-segment launch, then w2).

The reference engine has no MoE layer; this is the host-side grouping that its decode+GEMM
entry point (`nv_launch_split12_fused_gemm_async`, nvidia_kernels.cu:444) would be driven with
for a Mixtral-shaped layer: one call per expert with that expert's variable token count as B.
torch is used for the routing bookkeeping only (top-k, sort, gather, weighted scatter-add).
"""
from . import DeviceTensor12, gemm, lib, check, current_stream, _seg_array, _torch


class Expert:
    """w1 (gate), w3 (up): [n_ff, n_embd]; w2 (down): [n_embd, n_ff]; all DeviceTensor12."""

    def __init__(self, w1: DeviceTensor12, w3: DeviceTensor12, w2: DeviceTensor12):
        assert w1.M == w3.M == w2.K and w1.K == w3.K == w2.M
        self.w1, self.w3, self.w2 = w1, w3, w2


def route_top_k(router_logits, k=2):
    """softmax over the k largest logits per token -> (expert ids [T,k], weights [T,k] fp32)."""
    torch = _torch()
    top, idx = torch.topk(router_logits.float(), k, dim=-1)
    return idx, torch.softmax(top, dim=-1)


def moe_ffn(experts, X, expert_ids, weights, stream=None):
    """X bf16 bits [T, n_embd] (int16 tensor); returns fp32 [T, n_embd] = sum_j w[t,j] * FFN_{e[t,j]}(x_t)."""
    torch = _torch()
    st = current_stream() if stream is None else stream
    T, n = X.shape
    k = expert_ids.shape[1]
    n_ff = experts[0].w1.M
    flat_e = expert_ids.reshape(-1)
    order = torch.argsort(flat_e, stable=True)                     # (token, slot) pairs grouped per expert
    counts = torch.bincount(flat_e, minlength=len(experts)).tolist()
    tok = torch.div(order, k, rounding_mode="floor")
    Xg = X[tok].contiguous()                                       # [T*k, n] gathered rows
    wg = weights.reshape(-1)[order]
    out = torch.zeros((T, n), dtype=torch.float32, device=X.device)
    gate = torch.empty((max(counts), n_ff), dtype=torch.float32, device=X.device)
    up = torch.empty_like(gate)
    act = torch.empty((max(counts), n_ff), dtype=torch.int16, device=X.device)
    yd = torch.empty((max(counts), n), dtype=torch.float32, device=X.device)
    pos = 0
    for e, cnt in enumerate(counts):
        if cnt == 0:
            continue
        ex = experts[e]
        xs = Xg[pos:pos + cnt]
        # SiLU*mul in the GEMM's epilogue where the group is large enough to have such a kernel
        rc = lib.t12_gemm_swiglu(_seg_array([ex.w1.segment(None)]), _seg_array([ex.w3.segment(None)]), xs.data_ptr(),
                                 xs.stride(0), n, cnt, act.data_ptr(), n_ff, st)
        check(min(rc, 0), "t12_gemm_swiglu")
        if rc == 1:
            gemm([ex.w1, ex.w3], xs, outs=[gate[:cnt], up[:cnt]], stream=st)
            lib.launch_silu_mul_bf16_batch(gate.data_ptr(), up.data_ptr(), act.data_ptr(), n_ff, cnt, st)
        gemm([ex.w2], act[:cnt], outs=[yd[:cnt]], stream=st)
        out.index_add_(0, tok[pos:pos + cnt], yd[:cnt] * wg[pos:pos + cnt, None])
        pos += cnt
    return out
