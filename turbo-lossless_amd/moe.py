"""Mixture-of-experts SwiGLU FFN over split-12 experts: tokens grouped per expert, each group
through the fused decode+GEMM (w1|w3 as one two-segment launch, then w2).

The reference engine has no MoE layer; this is the host-side grouping that its decode+GEMM
entry point (`nv_launch_split12_fused_gemm_async`, nvidia_kernels.cu:444) would be driven with
for a Mixtral-shaped layer: one call per expert with that expert's variable token count as B.
torch is used for the routing bookkeeping only (top-k, sort, gather, weighted scatter-add).
"""
from . import DeviceTensor12, gemm, lib, check, _seg_array, _torch


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


_side_streams = {}


def _streams_for(device, n):
    """n side streams of the device (default priority), created once."""
    torch = _torch()
    key = (device.index if device.index is not None else torch.cuda.current_device(), n)
    if key not in _side_streams:
        _side_streams[key] = [torch.cuda.Stream(device=device) for _ in range(n)]
    return _side_streams[key]


def moe_ffn(experts, X, expert_ids, weights, stream=None, concurrency=2):
    """X bf16 bits [T, n_embd] (int16 tensor); returns fp32 [T, n_embd] = sum_j w[t,j] * FFN_{e[t,j]}(x_t).

    The experts' launch chains (w1|w3, SiLU*mul, w2) are independent of each other: with concurrency > 1 they are
    issued round-robin on that many side streams, so that one expert's weight stream starts under the tail of
    another's; the weighted scatter-add of all (token, expert) pairs follows as one operation on the caller's
    stream.  `stream`, when given, must be torch's current stream: the routing bookkeeping is torch operations."""
    torch = _torch()
    T, n = X.shape
    k = expert_ids.shape[1]
    n_ff = experts[0].w1.M
    flat_e = expert_ids.reshape(-1)
    order = torch.argsort(flat_e, stable=True)                     # (token, slot) pairs grouped per expert
    counts = torch.bincount(flat_e, minlength=len(experts)).tolist()
    tok = torch.div(order, k, rounding_mode="floor")
    Xg = X[tok].contiguous()                                       # [T*k, n] gathered rows
    wg = weights.reshape(-1)[order]
    main = torch.cuda.current_stream(X.device)
    if stream is not None and stream != main.cuda_stream:
        raise ValueError("moe_ffn works on torch's current stream: make the stream current instead of passing its handle")
    lanes = max(1, min(int(concurrency), sum(c > 0 for c in counts)))
    side = _streams_for(X.device, lanes) if lanes > 1 else [None]
    cap = max(counts)
    gate = [torch.empty((cap, n_ff), dtype=torch.float32, device=X.device) for _ in side]
    up = [torch.empty_like(g) for g in gate]
    act = [torch.empty((cap, n_ff), dtype=torch.int16, device=X.device) for _ in side]
    Y = torch.empty((T * k, n), dtype=torch.float32, device=X.device)      # every pair's FFN output, grouped like Xg
    if lanes > 1:
        ready = torch.cuda.Event()
        ready.record(main)
        for s in side:
            s.wait_event(ready)
    pos, turn = 0, 0
    for e, cnt in enumerate(counts):
        if cnt == 0:
            continue
        ex = experts[e]
        lane = turn % lanes
        turn += 1
        st = side[lane].cuda_stream if lanes > 1 else main.cuda_stream
        xs = Xg[pos:pos + cnt]
        # SiLU*mul in the GEMM's epilogue where the group is large enough to have such a kernel
        rc = lib.t12_gemm_swiglu(_seg_array([ex.w1.segment(None)]), _seg_array([ex.w3.segment(None)]), xs.data_ptr(),
                                 xs.stride(0), n, cnt, act[lane].data_ptr(), n_ff, st)
        check(min(rc, 0), "t12_gemm_swiglu")
        if rc == 1:
            gemm([ex.w1, ex.w3], xs, outs=[gate[lane][:cnt], up[lane][:cnt]], stream=st)
            lib.launch_silu_mul_bf16_batch(gate[lane].data_ptr(), up[lane].data_ptr(), act[lane].data_ptr(), n_ff, cnt, st)
        gemm([ex.w2], act[lane][:cnt], outs=[Y[pos:pos + cnt]], stream=st)
        pos += cnt
    if lanes > 1:
        for s in side:
            main.wait_stream(s)
    out = torch.zeros((T, n), dtype=torch.float32, device=X.device)
    out.index_add_(0, tok, Y * wg[:, None])                        # two addends per token: the order cannot matter
    return out
