"""Mixture-of-experts SwiGLU FFN over split-12 experts (a Mixtral-shaped layer).

The reference engine has no MoE layer; its decode+GEMM entry point (`nv_launch_split12_fused_gemm_async`,
nvidia_kernels.cu:444) would be called once per expert and projection with that expert's token count as B.  Here
the layer is the library's `t12_moe_ffn`: the (token, slot) pairs are grouped per expert on the GPU, gate|up (SwiGLU
in the epilogue) and down of all experts run as grouped decode+GEMM launches that read the rows per expert from the
device, and the weighted sum is taken in a fixed order; the host never waits.  torch
holds the buffers; `route_top_k` (top-k and softmax of the router logits) is the only torch arithmetic, and it is
not part of `moe_ffn`.
"""
from . import DeviceTensor12, Group, MoeExpert, lib, check, current_stream, _torch


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


class MoeLayer:
    """The experts of one layer as the table t12_moe_ffn takes, with a workspace that grows to the largest call."""

    def __init__(self, experts):
        self.experts = list(experts)
        self.n_ff, self.n_embd = self.experts[0].w1.M, self.experts[0].w1.K
        self.table = (MoeExpert * len(self.experts))()
        for i, e in enumerate(self.experts):
            assert (e.w1.M, e.w1.K) == (self.n_ff, self.n_embd)
            self.table[i].w1, self.table[i].w3, self.table[i].w2 = e.w1.segment(None), e.w3.segment(None), e.w2.segment(None)
        self.ws = None

    def workspace(self, T, k, device):
        need = lib.t12_moe_workspace_bytes(T, k, self.n_embd, self.n_ff, len(self.experts))
        if self.ws is None or self.ws.numel() < need or self.ws.device != device:
            self.ws = _torch().empty(need, dtype=_torch().uint8, device=device)
        return self.ws

    def __call__(self, X, expert_ids, weights, out=None, stream=None):
        """X bf16 bits [T, n_embd] (int16 tensor, rows may be strided); expert_ids [T, k] int32 / int64 and weights
        [T, k] fp32, contiguous; returns fp32 [T, n_embd] = sum_j w[t,j] * FFN_{e[t,j]}(x_t).  Nothing waits for the
        stream; the k ids of a token must be distinct.  An id outside the experts leaves its pair out of the sum:
        status() tells (it waits for the stream)."""
        torch = _torch()
        T, n = X.shape
        k = expert_ids.shape[1]
        assert n == self.n_embd and X.stride(1) == 1 and expert_ids.is_contiguous() and weights.is_contiguous()
        assert weights.dtype == torch.float32 and expert_ids.dtype in (torch.int32, torch.int64)
        if out is None:
            out = torch.empty((T, n), dtype=torch.float32, device=X.device)
        ws = self.workspace(T, k, X.device)
        st = current_stream() if stream is None else stream
        check(lib.t12_moe_ffn(self.table, len(self.experts), X.data_ptr(), X.stride(0), expert_ids.data_ptr(),
                              expert_ids.element_size(), weights.data_ptr(), T, k, n, self.n_ff, ws.data_ptr(), ws.numel(),
                              out.data_ptr(), out.stride(0), st), "t12_moe_ffn")
        self._last_stream = st
        return out

    def status(self):
        """Waits for the stream of the last call and raises T12Error if its routing met an id outside the experts (or
        a token that named one expert twice)."""
        if self.ws is not None:
            check(lib.t12_moe_status(self.ws.data_ptr(), getattr(self, "_last_stream", current_stream())), "t12_moe_status")


def moe_ffn(experts, X, expert_ids, weights, stream=None):
    """One call of a layer built on the spot (keep a MoeLayer to reuse the table and the workspace).  The workspace
    is a torch tensor released on return, so the work must be on torch's current stream."""
    if stream is not None and stream != current_stream():
        raise ValueError("moe_ffn works on torch's current stream: make the stream current, or keep a MoeLayer")
    return MoeLayer(experts)(X, expert_ids, weights, stream=stream)


def gemm_grouped(items, K, stream=None):
    """items: (DeviceTensor12, X int16 [B, K] rows strided, out fp32 [B, M]) per group -> one t12_gemm_grouped launch."""
    g = (Group * len(items))()
    for i, (w, X, out) in enumerate(items):
        g[i].seg = w.segment(out)
        g[i].seg.out_stride = out.stride(0) if out.shape[0] > 1 else w.M
        g[i].act_bf16 = X.data_ptr()
        g[i].act_stride = X.stride(0) if X.shape[0] > 0 else K
        g[i].B = X.shape[0]
    st = current_stream() if stream is None else stream
    check(lib.t12_gemm_grouped(g, len(items), K, st), "t12_gemm_grouped")
