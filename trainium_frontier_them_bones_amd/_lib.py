"""ctypes binding of the C-ABI library (include/tfb_kernels.h).

The library is the product path: if it has not been built, or a symbol is missing, loading
raises. There is no CPU or PyTorch fallback behind these entry points.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("TFB_LIB_PATH") or os.path.join(HERE, "libtfb_hip.so")  # override: another build of the same ABI

_vp = ctypes.c_void_p
_i = ctypes.c_int
_l = ctypes.c_long
_f = ctypes.c_float
_lp = ctypes.POINTER(ctypes.c_long)
_fp = ctypes.POINTER(ctypes.c_float)   # a HOST array of floats (tfb_ns5's coefficients)

# name -> argtypes (restype is always int status unless listed in _RESTYPE)
SIGNATURES = {
    "tfb_gemm_bf16": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _l, _vp],
    "tfb_gemm_bf16_scaled": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _l, _vp, _vp],
    "tfb_gemm_bf16_res": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "tfb_norm_bwd_blocks": [_l],
    "tfb_rmsnorm_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _f, _vp],
    "tfb_rmsnorm_fwd_q": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _l, _i, _f, _vp],
    "tfb_rmsnorm_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _l, _i, _vp],
    "tfb_rmsnorm_bwd_amax": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _l, _i, _vp],
    "tfb_norm_dw_finish": [_vp, _vp, _i, _l, _l, _i, _l, _i, _vp],
    "tfb_block_head_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _f, _vp],
    "tfb_block_head_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _vp],
    "tfb_mlp8_scale_scratch_floats": [_i],
    "tfb_mlp8_forward_scales": [_vp, _vp, _vp, _vp, _i, _i, _f, _f, _vp, _vp],
    "tfb_mlp8_backward_scales": [_vp, _vp, _vp, _vp, _l, _i, _vp],
    "tfb_mlp8_backward_scales_part": [_vp, _i, _vp, _vp, _i, _vp],
    "tfb_amax_scale": [_vp, _l, _f, _i, _i, _vp, _vp, _vp],
    "tfb_quant_fp8": [_vp, _vp, _f, _i, _vp, _l, _vp],
    "tfb_mlp8_precast": [_vp, _vp, _vp, _vp, _i, _i, _vp],
    "tfb_mlp8_refresh_layers": [_vp, _vp, _l, _i, _vp, _vp, _vp, _i, _i, _f, _f, _vp],
    "tfb_mlp8_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_mlp8_fwd_res": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_mlp8_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_mlp8_bwd_q": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _l, _i, _i, _vp],
    "tfb_gemm_fp8_tn": [_vp, _i, _vp, _i, _vp, _vp, _f, _vp, _l, _i, _i, _i, _i, _vp, _l, _vp],
    "tfb_mlp8_dw8": [_vp, _vp, _vp, _vp, _vp, _f, _vp, _vp, _l, _i, _i, _i, _i, _vp, _l, _vp, _vp],
    "tfb_attn_fwd": [_vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _i, _i, _i, _i, _f, _vp],
    "tfb_attn_fwd_band": [_vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _i, _i, _i, _i, _f, _i, _vp],
    "tfb_attn_bwd_band": [_vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _vp, _vp, _vp,
                          _i, _i, _i, _i, _f, _i, _vp],
    "tfb_attn_bwd": [_vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _vp, _i, _i, _i, _i,
                     _f, _vp],
    "tfb_attn_bwd_static": [_vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _i, _i, _i, _i,
                            _f, _vp],
    "tfb_attn_bwd_static_max_rows": [],
    "tfb_attn_bwd_rope": [_vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _lp, _vp, _vp, _vp, _vp,
                          _i, _i, _i, _i, _f, _vp],
    "tfb_qkv_rope_fwd": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "tfb_precast8": [_vp, _vp, _vp, _vp, _i, _i, _vp],
    "tfb_gemm_fp8": [_vp, _i, _vp, _vp, _vp, _f, _vp, _l, _i, _i, _vp],
    "tfb_gemm_fp8_res": [_vp, _vp, _vp, _vp, _f, _vp, _vp, _l, _i, _i, _vp],
    "tfb_relu2": [_vp, _vp, _vp, _l, _i, _vp],
    "tfb_rope": [_vp, _vp, _vp, _vp, _l, _i, _i, _i, _l, _l, _i, _vp],
    "tfb_rope_norm_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _i, _l, _l, _l, _f, _vp],
    "tfb_rope_norm_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _i, _l, _l, _l, _vp],
    "tfb_resmix_bwd_blocks": [_l],
    "tfb_resmix_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _vp],
    "tfb_embedding_fwd": [_vp, _i, _vp, _vp, _l, _i, _i, _vp],
    "tfb_embedding_bwd": [_vp, _i, _vp, _vp, _l, _i, _i, _vp],
    "tfb_embedding_bwd_scratch_ints": [_l, _i],
    "tfb_embedding_bwd_grouped": [_vp, _i, _vp, _vp, _l, _i, _i, _vp, _vp],
    "tfb_adamw": [_vp, _vp, _i, _vp, _vp, _vp, _l, _f, _f, _f, _f, _f, _f, _f, _vp],
    "tfb_fill_f32": [_vp, _f, _l, _vp],
    "tfb_loss_fwd": [_vp, _vp, _i, _vp, _vp, _vp, _l, _i, _f, _vp],
    "tfb_loss_fwd_bwd": [_vp, _vp, _i, _vp, _vp, _vp, _l, _i, _f, _vp],
    "tfb_mlp_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_mlp_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_gradnorm_scratch_floats": [],
    "tfb_gradnorm": [_vp, _l, _vp, _l, _f, _vp, _vp, _vp],
    "tfb_mix_tail_fwd": [_vp, _vp, _vp, _vp, _vp, _l, _i, _i, _f, _vp],
    "tfb_mix_tail_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_loss_row_weights": [_vp, _i, _vp, _l, _i, _i, _vp],
    "tfb_loss_bwd": [_vp, _vp, _i, _vp, _vp, _vp, _l, _i, _f, _vp],
    "tfb_loss_multi_fwd": [_vp, _vp, _i, _vp, _i, _f, _vp, _vp, _l, _i, _f, _vp],
    "tfb_loss_multi_bwd": [_vp, _vp, _i, _vp, _i, _f, _vp, _vp, _vp, _l, _i, _f, _vp],
    "tfb_lmhead_fwd": [_vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _f, _vp],
    "tfb_moe_max_rows": [_l, _i, _i],
    "tfb_moe_route": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _i, _vp],
    "tfb_moe_tables": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _l, _vp],
    "tfb_moe_tables_cap": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _l, _i, _i, _i, _l, _vp],
    "tfb_moe_gather": [_vp, _vp, _vp, _f, _vp, _vp, _l, _i, _vp],
    "tfb_moe_mlp8_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_moe_mlp8_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_moe_dw": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "tfb_moe_combine": [_vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_moe_combine_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_moe_combine_bwd_rowmax": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_moe_route_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _l, _i, _i, _i, _vp],
    "tfb_moe_route_bwd_aux": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _f, _f, _l, _i, _i, _i, _vp],
    "tfb_moe_aux_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_moe_mlp8_bwd_q": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _l, _i, _i, _vp],
    "tfb_moe_dw8": [_vp, _vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "tfb_moe_mlp_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_moe_mlp_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_moe_aux_seq_fwd": [_vp, _vp, _vp, _vp, _vp, _l, _l, _i, _i, _vp],
    "tfb_moe_route_bwd_aux_seq": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _f, _f, _vp, _f, _l, _l, _i, _i, _i, _vp],
    "tfb_moe_backward_scales": [_vp, _vp, _vp, _vp, _vp, _l, _i, _i, _vp],
    "tfb_moe_backward_scales_rowmax": [_vp, _vp, _vp, _vp, _i, _i, _vp],
    "tfb_moe_quant": [_vp, _vp, _vp, _i, _i, _vp, _l, _i, _vp],
    "tfb_ns5_workspace_bytes": [_i, _i, _i],
    "tfb_ns5": [_vp, _vp, _fp, _vp, _vp, _i, _i, _i, _i, _vp, _l, _vp],
    "tfb_mlp_dw_proj": [_vp, _vp, _vp, _l, _i, _i, _i, _i, _vp, _l, _vp],
}

_LONG_RESULT = {"tfb_gradnorm_scratch_floats", "tfb_attn_bwd_static_max_rows", "tfb_mlp8_scale_scratch_floats", "tfb_moe_max_rows", "tfb_embedding_bwd_scratch_ints", "tfb_ns5_workspace_bytes"}

STATUS = {0: "ok", 1: "unsupported shape", 2: "bad argument", 3: "kernel launch failed", 4: "workspace too small"}


class TfbError(RuntimeError):
    def __init__(self, fn, status):
        self.status = status
        super().__init__("%s returned %d (%s)" % (fn, status, STATUS.get(status, "?")))


_LIB = None


def lib():
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "HIP extension %s is not built; run `python -m trainium_frontier_them_bones_amd.build`" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, args in SIGNATURES.items():
            fn = getattr(L, name)  # AttributeError if the symbol is missing
            fn.argtypes = args
            fn.restype = _l if name in _LONG_RESULT else _i
        _LIB = L
    return _LIB


# name -> list: when an entry point is listed here every call is bracketed by events on torch's current stream
# (the stream the kernels are launched on) and (start, end, name, args) appended; the key "*" takes every entry point
# not listed by name. Used by the benchmark only.
TIMED = {}


def call(name, *args):
    rec = None
    if TIMED:
        rec = TIMED.get(name)
        if rec is None:
            rec = TIMED.get("*")
    if rec is None:
        st = getattr(lib(), name)(*args)
    else:
        import torch
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        st = getattr(lib(), name)(*args)
        e.record()
        rec.append((s, e, name, args))
    if st != 0:
        raise TfbError(name, st)
