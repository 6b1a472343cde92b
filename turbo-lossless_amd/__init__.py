"""turbo12 for MI355X: ctypes face of libturbo12.so (the C ABI in include/t12_abi.h).

The library is the product; this module only marshals pointers.  torch is used
for device memory and streams.  There is no CPU fallback: if the HIP library is
missing, importing this module fails.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libturbo12.so")
MAX_SEGMENTS = 8

if not os.path.exists(LIB_PATH):
    raise ImportError(
        "libturbo12.so is not built: run `python turbo-lossless_amd/build.py` "
        "(hipcc --offload-arch=gfx950). There is no CPU fallback.")

lib = C.CDLL(LIB_PATH)


class Segment(C.Structure):
    """Mirror of T12Segment (include/t12_abi.h)."""
    _fields_ = [("sm", C.c_void_p), ("gr", C.c_void_p), ("row_off", C.c_void_p), ("cols", C.c_void_p),
                ("correct", C.c_void_p), ("wrong", C.c_void_p), ("out", C.c_void_p),
                ("M", C.c_int32), ("base_exp", C.c_int32), ("out_stride", C.c_int32), ("reserved", C.c_int32)]


class PatchBatchDesc(C.Structure):
    _fields_ = [("row_offsets", C.c_void_p), ("patch_cols", C.c_void_p), ("patch_correct", C.c_void_p),
                ("patch_wrong", C.c_void_p), ("activations", C.c_void_p), ("output", C.c_void_p), ("M", C.c_int)]


class Group(C.Structure):
    """Mirror of T12Group (include/t12_abi.h)."""
    _fields_ = [("seg", Segment), ("act_bf16", C.c_void_p), ("act_stride", C.c_int), ("B", C.c_int)]


class MoeExpert(C.Structure):
    """Mirror of T12MoeExpert (include/t12_abi.h)."""
    _fields_ = [("w1", Segment), ("w3", Segment), ("w2", Segment)]


class GemmPartials(C.Structure):
    """Mirror of T12GemmPartials (include/t12_abi.h)."""
    _fields_ = [("ws", C.c_void_p), ("nsplit", C.c_int), ("ld", C.c_int), ("split_stride", C.c_size_t)]


_vp, _i = C.c_void_p, C.c_int
_SIGS = {
    "t12_version": (C.c_char_p, []),
    "t12_last_error": (C.c_char_p, []),
    "t12_pack_histogram": (_i, [_vp, C.c_size_t, _vp, _vp]),
    "t12_pack_base_exp": (_i, [C.POINTER(C.c_uint64)]),
    "t12_pack_planes": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "t12_pack_row_offsets": (_i, [_vp, _i, _vp, _vp]),
    "t12_pack_escapes": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "t12_gemv": (_i, [C.POINTER(Segment), _i, _vp, _i, _vp]),
    "t12_synth_normal_bf16": (_i, [_vp, C.c_size_t, C.c_uint64, C.c_float, C.c_float, C.c_float, _vp]),
    "t12_fill_f32": (_i, [_vp, C.c_size_t, C.c_float, _vp]),
    # glue launchers (reference names; void return)
    "t12_tune_attention": (_i, [_i]),
    "launch_rope_init": (None, [_i, C.c_float]),
    "launch_rope_scaling": (None, [C.c_float] * 4),
    "t12_rope_freqs": (None, [_i] + [C.c_float] * 5 + [_vp]),
    "launch_embed_lookup": (None, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "launch_rms_norm_bf16_batch": (None, [_vp, _vp, _vp, _i, C.c_float, _i, _vp]),
    "launch_add_rms_norm_bf16_batch": (None, [_vp, _vp, _vp, _vp, _i, C.c_float, _i, _vp]),
    "launch_silu_mul_bf16_batch": (None, [_vp, _vp, _vp, _i, _i, _vp]),
    "launch_add_batch": (None, [_vp, _vp, _i, _i, _vp]),
    "launch_rope_batch": (None, [_vp, _vp, _vp, _i, _i, _i, _i, _i, C.c_float, _i, _vp]),
    "launch_store_kv_batch": (None, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "launch_rope_store_kv": (None, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, C.c_float, _vp]),
    "launch_rope_store_kv_batch": (None, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, C.c_float, _i, _vp]),
    "launch_rope_store_attention": (None, [_vp] * 9 + [_i, _i, _i, _i, C.c_float, C.c_float, _i, _i, _vp]),
    "launch_rope_store_attention_partials": (None, [_vp] * 9 + [_i, _i, _i, _i, C.c_float, C.c_float, _i, _vp, _i,
                                                    C.c_size_t, _i, _i, _vp]),
    "launch_rope_store_attention_regions": (None, [_vp] * 9 + [_i, _i, _i, _i, C.c_float, C.c_float, _i, _i, _i, _vp]),
    "launch_rope_store_attention_partials_regions": (None, [_vp] * 9 + [_i, _i, _i, _i, C.c_float, C.c_float, _i, _vp, _i,
                                                            C.c_size_t, _i, _i, _i, _vp]),
    "launch_attention_all_heads": (None, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, C.c_float, _vp]),
    "launch_flash_attention": (None, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, C.c_float, _vp]),
    "launch_attention_all_heads_batch": (None, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, C.c_float, _i, _i, _vp]),
    "launch_flash_attention_batch": (None, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, C.c_float, _i, _i, _vp]),
    "launch_argmax": (None, [_vp, _vp, _i, _vp]),
    "launch_argmax_batch": (None, [_vp, _vp, _i, _i, _vp]),
    # engine (C face of model.h / inference.h / sampler.h)
    "t12_engine_load": (_vp, [C.c_char_p, _i]),
    "t12_engine_check_dir": (_i, [C.c_char_p, C.c_char_p, C.c_size_t]),
    "t12_engine_weight_tables": (_i, [_vp, _i, _i, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_i)]),
    "t12_engine_create_synthetic": (_vp, [_i, _i, _i, _i, _i, _i, _i, C.c_float, C.c_float, C.c_uint64, _i, C.c_float]),
    "t12_engine_save": (_i, [_vp, C.c_char_p]),
    "t12_engine_free_model": (None, [_vp]),
    "t12_engine_create_state": (_vp, [_vp, _i, _i]),
    "t12_engine_create_state_per_sequence": (_vp, [_vp, _i, _i]),
    "t12_engine_prefill": (_i, [_vp, _i, C.POINTER(C.c_int), _i]),
    "t12_engine_decode_all": (_i, [_vp, _i, C.POINTER(C.c_int)]),
    "t12_engine_free_state": (None, [_vp]),
    "t12_engine_forward": (_i, [_vp, C.POINTER(C.c_int)]),
    "t12_engine_logits": (_vp, [_vp]),
    "t12_engine_stream": (_vp, [_vp]),
    "t12_engine_max_seq": (_i, [_vp]),
    "t12_engine_set_positions": (None, [_vp, C.POINTER(C.c_int)]),
    "t12_engine_get_positions": (None, [_vp, C.POINTER(C.c_int)]),
    "t12_engine_sample": (_i, [_vp, C.POINTER(C.c_int)]),
    "t12_engine_generate": (_i, [_vp, C.POINTER(C.c_int), _i, _i, C.POINTER(C.c_int)]),
    "t12_engine_decode": (_i, [_vp, _i, _i, C.POINTER(C.c_int)]),
    "t12_engine_decode_until": (_i, [_vp, _i, _i, C.POINTER(C.c_int)]),
    "t12_engine_sync": (_i, [_vp]),
    "t12_engine_shift_context": (_i, [_vp, _i, _i, _i]),
    "t12_engine_chat_turn": (_i, [_vp, C.POINTER(C.c_int), C.POINTER(C.c_int), _i, _i, _i, _i, _i, C.POINTER(C.c_int),
                                  C.POINTER(C.c_int)]),
    "t12_engine_prefill_rows": (_i, [_vp, C.POINTER(C.c_int), _i, _i]),
    "t12_tokenizer_load": (_vp, [C.c_char_p]),
    "t12_tokenizer_free": (None, [_vp]),
    "t12_tokenizer_info": (_i, [_vp, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "t12_tokenizer_type": (_i, [_vp]),
    "t12_tokenizer_special": (_i, [_vp, _i, C.c_char_p, C.c_size_t, C.POINTER(C.c_int)]),
    "t12_tokenizer_add_special": (_i, [_vp, C.c_char_p, _i]),
    "t12_tokenizer_encode": (_i, [_vp, C.c_char_p, C.c_size_t, C.POINTER(C.c_int), _i]),
    "t12_tokenizer_decode": (_i, [_vp, C.POINTER(C.c_int), _i, C.c_char_p, C.c_size_t]),
    "t12_tokenizer_decode_one": (_i, [_vp, _i, C.c_char_p, C.c_size_t]),
    "t12_engine_weight": (_i, [_vp, _i, _i, C.POINTER(Segment), C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "t12_gemv_add": (_i, [C.POINTER(Segment), _vp, _i, _vp, _vp]),
    "t12_gemv_swiglu": (_i, [C.POINTER(Segment), C.POINTER(Segment), _vp, _i, _vp, _vp]),
    "t12_gemv_norm": (_i, [C.POINTER(Segment), _i, _vp, _vp, _vp, C.c_float, _vp, _i, _vp]),
    "t12_gemv_swiglu_norm": (_i, [C.POINTER(Segment), C.POINTER(Segment), _vp, _vp, _vp, C.c_float, _vp, _i, _vp, _vp]),
    "t12_gemv_batch": (_i, [C.POINTER(Segment), _i, _vp, _i, _i, _i, _i, _vp]),
    "launch_split12_batch4_async": (_i, [_vp] * 2 + [_i] + [_vp] * 4 + [_vp] * 3 + [_vp] * 4 + [_i, _i, _vp]),
    "launch_split12_batch8_async": (_i, [_vp] * 2 + [_i] + [_vp] * 8 + [_vp] * 3 + [_vp] * 8 + [_i, _i, _vp]),
    "nv_launch_split12_fused_gemm_async": (_i, [_vp, _vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "nv_launch_patches_batch_async": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _i, _i, _vp]),
    "nv_launch_split12_cublas_batch_async": (_i, [_vp, _vp, _i, _vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _vp]),
    "t12_gemm": (_i, [C.POINTER(Segment), _i, _vp, _i, _i, _i, _i, _vp]),
    "t12_gemm_noalloc": (_i, [C.POINTER(Segment), _i, _vp, _i, _i, _i, _i, _vp]),
    "t12_gemm_grouped": (_i, [C.POINTER(Group), _i, _i, _vp]),
    "t12_release_stream": (_i, [_vp]),
    "t12_moe_workspace_bytes": (C.c_size_t, [_i, _i, _i, _i, _i]),
    "t12_moe_ffn": (_i, [C.POINTER(MoeExpert), _i, _vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _vp, C.c_size_t, _vp, _i, _vp]),
    "t12_moe_status": (_i, [_vp, _vp]),
    "t12_probe_clock": (_i, [_i, _i, _i, C.POINTER(C.c_double), C.POINTER(C.c_double), _vp]),
    "t12_probe_launch_gap": (_i, [_i, _i, C.POINTER(C.c_double), _vp]),
    "t12_gemm_swiglu": (_i, [C.POINTER(Segment), C.POINTER(Segment), _vp, _i, _i, _i, _vp, _i, _vp]),
    "t12_gemm_deferred": (_i, [C.POINTER(Segment), _i, _vp, _i, _i, _i, _i, C.POINTER(GemmPartials), _vp]),
    "launch_sum_add_rms_norm_bf16_batch": (None, [_vp, _vp, _i, C.c_size_t, _i, _vp, _vp, _vp, _i, C.c_float, _i, _vp]),
    "t12_util_copy_i32": (_i, [_vp, _vp, _i, _vp]),
    "t12_decompress": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "launch_split12_v2_async": (_i, [_vp, _vp, _i, _vp, _vp, _i, _i, _vp]),
    "launch_split12_v2_dual_async": (_i, [_vp, _vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _vp]),
    "launch_patches_v2_async": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "launch_patches_v2": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i]),
    "launch_patches_b1_batched_async": (_i, [_vp, C.POINTER(PatchBatchDesc), _i, _i, _vp]),
}
for _name, (_res, _args) in _SIGS.items():
    _fn = getattr(lib, _name)
    _fn.restype, _fn.argtypes = _res, _args


class T12Error(RuntimeError):
    pass


def check(rc: int, what: str = "") -> None:
    if rc != 0:
        raise T12Error("%s failed (%d): %s" % (what, rc, lib.t12_last_error().decode()))


def _count(n: int, what: str) -> int:
    """A t12_engine_* result that is a count when >= 0 and a T12_E* code otherwise."""
    if n < 0:
        raise T12Error("%s failed (%d): %s" % (what, n, lib.t12_last_error().decode()))
    return n


def _torch():
    import torch
    return torch


def current_stream() -> int:
    return _torch().cuda.current_stream().cuda_stream


def _dp(t):
    return None if t is None else t.data_ptr()


class DeviceTensor12:
    """A split-12 tensor resident in HBM: the planes and the CSR escape list."""

    def __init__(self, M, K, base_exp, sm, gr, row_off=None, cols=None, correct=None, wrong=None):
        self.M, self.K, self.base_exp = int(M), int(K), int(base_exp)
        self.sm, self.gr = sm, gr
        self.row_off, self.cols, self.correct, self.wrong = row_off, cols, correct, wrong

    @classmethod
    def from_packed(cls, p, device="cuda"):
        """Upload the arrays a packer produced (anything with .sm .gr .row_off .cols .correct .wrong)."""
        torch = _torch()

        def up(a):
            a = np.ascontiguousarray(a)
            if a.size == 0:
                return torch.zeros(1, dtype=getattr(torch, str(a.dtype)), device=device)[:0]
            return torch.from_numpy(a).to(device)

        return cls(p.M, p.K, p.base_exp, up(p.sm), up(p.gr), up(p.row_off), up(p.cols), up(p.correct), up(p.wrong))

    @property
    def P(self):
        return 0 if self.cols is None else int(self.cols.numel())

    def segment(self, out, patched=True) -> Segment:
        use = patched and self.row_off is not None and self.P > 0   # no escapes: no list
        return Segment(_dp(self.sm), _dp(self.gr), _dp(self.row_off) if use else None,
                       _dp(self.cols) if use else None, _dp(self.correct) if use else None,
                       _dp(self.wrong) if use else None, _dp(out), self.M, self.base_exp,
                       int(out.stride(0)) if (out is not None and out.dim() == 2) else 0, 0)


def _seg_array(segs):
    arr = (Segment * len(segs))(*segs)
    return arr


def gemv(tensors, act, outs=None, patched=True, stream=None):
    """Fused decode-GEMV (B = 1) over one or more tensors sharing `act` (bf16 [K])."""
    torch = _torch()
    if isinstance(tensors, DeviceTensor12):
        tensors = [tensors]
    K = tensors[0].K
    if outs is None:
        outs = [torch.empty(t.M, dtype=torch.float32, device=act.device) for t in tensors]
    segs = _seg_array([t.segment(o, patched) for t, o in zip(tensors, outs)])
    st = current_stream() if stream is None else stream
    check(lib.t12_gemv(segs, len(tensors), act.data_ptr(), K, st), "t12_gemv")
    return outs


def gemm(tensors, X, outs=None, patched=True, stream=None):
    """Fused decode+GEMM: X is bf16 [B, K] (row stride = X.stride(0)); returns fp32 [B, M] per tensor."""
    torch = _torch()
    if isinstance(tensors, DeviceTensor12):
        tensors = [tensors]
    B, K = X.shape
    assert K == tensors[0].K and X.stride(1) == 1
    if outs is None:
        outs = [torch.empty((B, t.M), dtype=torch.float32, device=X.device) for t in tensors]
    stride = outs[0].stride(0)      # every segment carries its own stride; this is the default
    segs = _seg_array([t.segment(o, patched) for t, o in zip(tensors, outs)])
    st = current_stream() if stream is None else stream
    check(lib.t12_gemm(segs, len(tensors), X.data_ptr(), X.stride(0), stride, K, B, st), "t12_gemm")
    return outs


def decompress(t: DeviceTensor12, patched=True, out=None, stream=None):
    torch = _torch()
    if out is None:
        out = torch.empty((t.M, t.K), dtype=torch.int16, device=t.sm.device)
    st = current_stream() if stream is None else stream
    has = t.row_off is not None and t.P > 0
    check(lib.t12_decompress(_dp(t.sm), _dp(t.gr), t.base_exp, _dp(t.row_off) if has else None,
                             _dp(t.cols) if has else None, _dp(t.correct) if has else None,
                             out.data_ptr(), t.M, t.K, int(patched), st), "t12_decompress")
    return out


def find_base_exp_device(w, stream=None) -> int:
    """split12_find_base_exp on a bf16 matrix resident in HBM."""
    torch = _torch()
    st = current_stream() if stream is None else stream
    hist = torch.empty(256, dtype=torch.int64, device=w.device)
    check(lib.t12_pack_histogram(w.data_ptr(), w.numel(), hist.data_ptr(), st), "t12_pack_histogram")
    h = hist.cpu().numpy().astype(np.uint64)       # synchronises
    return int(lib.t12_pack_base_exp(h.ctypes.data_as(C.POINTER(C.c_uint64))))


def pack_device(w, base_exp=None, stream=None) -> DeviceTensor12:
    """Pack a bf16 matrix [M, K] (torch.bfloat16 or int16 bits, on the GPU) into split-12 on the GPU."""
    torch = _torch()
    assert w.dim() == 2 and w.is_contiguous() and w.element_size() == 2
    M, K = w.shape
    st = current_stream() if stream is None else stream
    if base_exp is None:
        base_exp = find_base_exp_device(w, st)
    n = M * K
    dev = w.device
    sm = torch.empty(n, dtype=torch.uint8, device=dev)
    gr = torch.empty((n + 1) // 2, dtype=torch.uint8, device=dev)
    cnt = torch.empty(M, dtype=torch.int32, device=dev)
    row_off = torch.empty(M + 1, dtype=torch.int32, device=dev)
    check(lib.t12_pack_planes(w.data_ptr(), M, K, base_exp, sm.data_ptr(), gr.data_ptr(), cnt.data_ptr(), st),
          "t12_pack_planes")
    check(lib.t12_pack_row_offsets(cnt.data_ptr(), M, row_off.data_ptr(), st), "t12_pack_row_offsets")
    P = int(row_off[M].item())                      # synchronises
    cols = torch.empty(P, dtype=torch.int32, device=dev)
    correct = torch.empty(P, dtype=torch.int16, device=dev)
    wrong = torch.empty(P, dtype=torch.int16, device=dev)
    if P:
        check(lib.t12_pack_escapes(w.data_ptr(), M, K, base_exp, row_off.data_ptr(), cols.data_ptr(),
                                   correct.data_ptr(), wrong.data_ptr(), st), "t12_pack_escapes")
    return DeviceTensor12(M, K, base_exp, sm, gr, row_off, cols, correct, wrong)


# ------------------------------------------------------------------ engine
class Engine:
    """The engine's load / forward / sample / generate API (include/turbo/*.h) through its C face."""

    def __init__(self, model_handle, batch=1, per_sequence=0):
        """per_sequence = N > 0: batch independent sequences, each with its own KV cache of N positions
        (create_inference_state_per_sequence); 0: the reference's one shared cache region."""
        if not model_handle:
            raise T12Error("model could not be loaded/created")
        self.model = model_handle
        self.batch = batch
        self.state = self._make_state(batch, per_sequence)

    def _make_state(self, batch, per_sequence):
        if per_sequence:
            st = lib.t12_engine_create_state_per_sequence(self.model, batch, int(per_sequence))
            if not st:
                raise T12Error("per-sequence KV cache could not be created")
            return st
        st = lib.t12_engine_create_state(self.model, batch, 0)
        if not st:
            raise T12Error("inference state could not be created: %s" % lib.t12_last_error().decode())
        return st

    @classmethod
    def load(cls, path, batch=1, device=0, per_sequence=0):
        return cls(lib.t12_engine_load(os.fsencode(path), device), batch, per_sequence)

    @classmethod
    def synthetic(cls, cfg, seed=4000, max_seq=2048, batch=1, p_outlier=3e-4, per_sequence=0):
        h = lib.t12_engine_create_synthetic(cfg["n_vocab"], cfg["n_embd"], cfg["n_head"], cfg["n_head_kv"],
                                            cfg["n_layer"], cfg["n_ff"], cfg.get("n_ctx", max_seq),
                                            cfg.get("rope_theta", 500000.0), cfg.get("rms_norm_eps", 1e-5), seed,
                                            max_seq, p_outlier)
        return cls(h, batch, per_sequence)

    def new_state(self, batch, per_sequence=0):
        """A second InferenceState on the same model (shared-region states share the model's KV cache)."""
        e = Engine.__new__(Engine)
        e.model, e.batch = self.model, batch
        e.state = e._make_state(batch, per_sequence)
        e._borrowed = True
        return e

    def prefill(self, seq, tokens):
        """Batched prompt pass of sequence seq (rows = prompt tokens, up to batch at a time)."""
        arr = (C.c_int * max(len(tokens), 1))(*[int(t) for t in tokens])
        check(lib.t12_engine_prefill(self.state, int(seq), arr, len(tokens)), "prefill")

    def decode_all(self, max_tokens):
        """max_tokens greedy steps from the current logits; ids of every sequence as [steps][batch]."""
        out = (C.c_int * max(max_tokens * self.batch, 1))()
        n = _count(lib.t12_engine_decode_all(self.state, max_tokens, out), "decode_all")
        return [list(out[t * self.batch:(t + 1) * self.batch]) for t in range(n)]

    def save(self, path):
        check(lib.t12_engine_save(self.model, os.fsencode(path)), "save_model")

    def set_positions(self, pos):
        arr = (C.c_int * self.batch)(*[int(p) for p in pos])
        lib.t12_engine_set_positions(self.state, arr)

    def positions(self):
        arr = (C.c_int * self.batch)()
        lib.t12_engine_get_positions(self.state, arr)
        return list(arr)

    def forward(self, tokens):
        arr = (C.c_int * self.batch)(*[int(t) for t in tokens])
        check(lib.t12_engine_forward(self.state, arr), "forward")

    def sync(self):
        check(lib.t12_engine_sync(self.state), "stream sync")

    def logits(self, n_vocab):
        """fp32 [batch, n_vocab] view of the device logits (synchronises the engine stream first)."""
        torch = _torch()
        self.sync()
        ptr = lib.t12_engine_logits(self.state)
        n = self.batch * n_vocab
        out = torch.empty((self.batch, n_vocab), dtype=torch.float32, device="cuda")
        rc = _hip_memcpy_d2d(out.data_ptr(), ptr, n * 4)
        if rc:
            raise T12Error("hipMemcpy failed (%d)" % rc)
        return out

    def sample(self):
        arr = (C.c_int * self.batch)()
        check(lib.t12_engine_sample(self.state, arr), "sample")
        return list(arr)

    def generate(self, prompt, max_tokens):
        p = (C.c_int * len(prompt))(*[int(t) for t in prompt])
        out = (C.c_int * max(max_tokens, 1))()
        n = _count(lib.t12_engine_generate(self.state, p, len(prompt), max_tokens, out), "generate")
        return list(out[:n])

    def decode(self, max_tokens, stop_on_eos=False):
        """Up to max_tokens greedy steps (sample, forward) from the current logits; ids of sequence 0."""
        out = (C.c_int * max(max_tokens, 1))()
        n = _count(lib.t12_engine_decode(self.state, max_tokens, int(stop_on_eos), out), "decode")
        return list(out[:n])

    def decode_until(self, max_tokens, stop_id):
        """Greedy steps until sequence 0 samples stop_id (not returned; -1: never) or max_tokens."""
        out = (C.c_int * max(max_tokens, 1))()
        n = _count(lib.t12_engine_decode_until(self.state, max_tokens, int(stop_id), out), "decode_until")
        return list(out[:n])

    def shift_context(self, current_pos, discard, seq=0):
        """Cache rows [discard, current_pos) of sequence seq move to the front (engine/main.cpp:147-173)."""
        check(lib.t12_engine_shift_context(self.state, int(seq), int(current_pos), int(discard)), "shift_context")

    def prefill_rows(self, tokens, rows):
        """Prompt pass of a batch-1 engine, `rows` tokens per pass (a helper state lends its buffers)."""
        arr = (C.c_int * max(len(tokens), 1))(*[int(t) for t in tokens])
        check(lib.t12_engine_prefill_rows(self.state, arr, len(tokens), int(rows)), "prefill_rows")

    def chat_turn(self, current_pos, tokens, max_tokens, bos_id, eos_id, prompt_rows=1):
        """One interactive turn (engine/main.cpp:139-213) -> (generated ids, new current_pos, rows discarded)."""
        pos, dropped = C.c_int(int(current_pos)), C.c_int(0)
        arr = (C.c_int * max(len(tokens), 1))(*[int(t) for t in tokens])
        out = (C.c_int * max(max_tokens, 1))()
        n = _count(lib.t12_engine_chat_turn(self.state, C.byref(pos), arr, len(tokens), int(max_tokens), int(bos_id),
                                            int(eos_id), int(prompt_rows), C.byref(dropped), out), "chat_turn")
        return list(out[:n]), pos.value, dropped.value

    def weight(self, layer, which):
        seg, K, P = Segment(), C.c_int(), C.c_int()
        check(lib.t12_engine_weight(self.model, layer, which, C.byref(seg), C.byref(K), C.byref(P)), "engine_weight")
        return seg, K.value, P.value

    def weight_tables(self, layer, which):
        """Device pointers (row_base, vals, nonempty_rows) and the number of non-empty rows."""
        rb, vals, ne, n = _vp(), _vp(), _vp(), C.c_int()
        check(lib.t12_engine_weight_tables(self.model, layer, which, C.byref(rb), C.byref(vals), C.byref(ne), C.byref(n)),
              "engine_weight_tables")
        return rb.value, vals.value, ne.value, n.value

    def close(self):
        if self.state:
            lib.t12_engine_free_state(self.state)
            self.state = None
        if self.model and not getattr(self, "_borrowed", False):
            lib.t12_engine_free_model(self.model)
        self.model = None


_hip = None


def _hip_memcpy_d2d(dst, src, nbytes):
    global _hip
    if _hip is None:
        _hip = C.CDLL("libamdhip64.so")
        _hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        _hip.hipMemcpy.restype = C.c_int
    return _hip.hipMemcpy(dst, src, nbytes, 3)   # hipMemcpyDeviceToDevice


def check_model_dir(path) -> str:
    """'' when the directory is consistent, else the loader's first finding (host only, no GPU)."""
    buf = C.create_string_buffer(512)
    return "" if lib.t12_engine_check_dir(os.fsencode(path), buf, 512) == 0 else (buf.value.decode() or "inconsistent")


class Tokenizer:
    """The engine's tokenizer (include/turbo/tokenizer.h: sentencepiece BPE model or byte-level BPE tables) through
    its C face; text is bytes."""

    def __init__(self, model_dir):
        self.handle = lib.t12_tokenizer_load(os.fsencode(model_dir))
        if not self.handle:
            raise T12Error("no tokenizer in %s (tokenizer.model, or vocab.bin + merges.bin)" % model_dir)
        b, e, v = C.c_int(), C.c_int(), C.c_int()
        lib.t12_tokenizer_info(self.handle, C.byref(b), C.byref(e), C.byref(v))
        self.bos_id, self.eos_id, self.vocab_size = b.value, e.value, v.value
        self.type = lib.t12_tokenizer_type(self.handle)

    def special_tokens(self) -> list:
        """[(text bytes, id)] in matching order (longest first)."""
        out, buf, tid = [], C.create_string_buffer(1024), C.c_int()
        for i in range(lib.t12_tokenizer_special(self.handle, -1, None, 0, None)):
            lib.t12_tokenizer_special(self.handle, i, buf, 1024, C.byref(tid))
            out.append((buf.value, tid.value))
        return out

    def add_special(self, text: bytes, tid: int):
        check(lib.t12_tokenizer_add_special(self.handle, bytes(text), int(tid)), "add_special")

    def tokenize(self, text) -> list:
        data = text.encode("utf-8") if isinstance(text, str) else bytes(text)
        cap = len(data) + 8
        out = (C.c_int * cap)()
        n = lib.t12_tokenizer_encode(self.handle, data, len(data), out, cap)
        if n < 0:
            raise T12Error("tokenize failed")
        if n > cap:
            out = (C.c_int * n)()
            n = lib.t12_tokenizer_encode(self.handle, data, len(data), out, n)
        return list(out[:n])

    def _text(self, fn, *args) -> bytes:
        n = fn(self.handle, *args, None, 0)
        if n < 0:
            raise T12Error("detokenize failed")
        buf = C.create_string_buffer(max(n, 1))
        fn(self.handle, *args, buf, n)
        return buf.raw[:n]

    def detokenize(self, ids) -> bytes:
        arr = (C.c_int * max(len(ids), 1))(*[int(t) for t in ids])
        return self._text(lib.t12_tokenizer_decode, arr, len(ids))

    def detokenize_one(self, tid) -> bytes:
        return self._text(lib.t12_tokenizer_decode_one, int(tid))

    def close(self):
        if self.handle:
            lib.t12_tokenizer_free(self.handle)
            self.handle = None
