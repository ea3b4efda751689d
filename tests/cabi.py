"""ctypes mirror of include/cc1d.h, used by the tests to call the C ABI directly (no
torch extension in between).  Field order and types must match the header exactly."""
import ctypes as C

import torch

F32, F16, BF16 = 0, 1, 2
DTYPES = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

i32, i64, vp = C.c_int32, C.c_int64, C.c_void_p


class FwdParams(C.Structure):
    _fields_ = [
        ("batch", i32), ("dim", i32), ("seqlen", i32), ("width", i32),
        ("x_dtype", i32), ("w_dtype", i32), ("silu", i32), ("reserved0", i32),
        ("x", vp), ("x_stride_b", i64), ("x_stride_c", i64), ("x_stride_l", i64),
        ("weight", vp), ("w_stride_c", i64), ("w_stride_w", i64),
        ("bias", vp),
        ("out", vp), ("out_stride_b", i64), ("out_stride_c", i64), ("out_stride_l", i64),
        ("seq_idx", vp),
        ("initial_states", vp), ("init_stride_b", i64), ("init_stride_c", i64), ("init_stride_l", i64),
        ("final_states", vp), ("final_stride_b", i64), ("final_stride_c", i64), ("final_stride_l", i64),
    ]


class BwdParams(C.Structure):
    _fields_ = [
        ("batch", i32), ("dim", i32), ("seqlen", i32), ("width", i32),
        ("x_dtype", i32), ("w_dtype", i32), ("silu", i32), ("overwrite_dweight", i32),
        ("x", vp), ("x_stride_b", i64), ("x_stride_c", i64), ("x_stride_l", i64),
        ("weight", vp), ("w_stride_c", i64), ("w_stride_w", i64),
        ("bias", vp),
        ("dout", vp), ("dout_stride_b", i64), ("dout_stride_c", i64), ("dout_stride_l", i64),
        ("seq_idx", vp),
        ("initial_states", vp), ("init_stride_b", i64), ("init_stride_c", i64), ("init_stride_l", i64),
        ("dfinal_states", vp), ("dfinal_stride_b", i64), ("dfinal_stride_c", i64), ("dfinal_stride_l", i64),
        ("dx", vp), ("dx_stride_b", i64), ("dx_stride_c", i64), ("dx_stride_l", i64),
        ("dweight", vp), ("dw_stride_c", i64), ("dw_stride_w", i64),
        ("dbias", vp),
        ("dinitial_states", vp), ("dinit_stride_b", i64), ("dinit_stride_c", i64), ("dinit_stride_l", i64),
    ]


class UpdateParams(C.Structure):
    _fields_ = [
        ("batch", i32), ("dim", i32), ("seqlen", i32), ("width", i32),
        ("state_len", i32), ("state_batch", i32),
        ("x_dtype", i32), ("w_dtype", i32), ("silu", i32), ("reserved0", i32),
        ("x", vp), ("x_stride_b", i64), ("x_stride_c", i64), ("x_stride_l", i64),
        ("conv_state", vp), ("state_stride_b", i64), ("state_stride_c", i64), ("state_stride_l", i64),
        ("weight", vp), ("w_stride_c", i64), ("w_stride_w", i64),
        ("bias", vp),
        ("out", vp), ("out_stride_b", i64), ("out_stride_c", i64), ("out_stride_l", i64),
        ("cache_seqlens", vp), ("conv_state_indices", vp),
    ]


class VarlenParams(C.Structure):
    _fields_ = [
        ("batch", i32), ("dim", i32), ("state_len", i32), ("x_dtype", i32),
        ("cu_seqlens_is_int64", i32), ("reserved0", i32),
        ("total_tokens", i64),
        ("x", vp), ("x_stride_t", i64), ("x_stride_c", i64),
        ("cu_seqlens", vp),
        ("states", vp), ("states_stride_b", i64), ("states_stride_c", i64), ("states_stride_l", i64),
    ]


def _ptr(t):
    return None if t is None else t.data_ptr()


def _set3(p, prefix, ptr_name, t):
    setattr(p, ptr_name, _ptr(t))
    if t is not None:
        for ax, name in enumerate(("b", "c", "l")):
            setattr(p, f"{prefix}_stride_{name}", t.stride(ax))


def fwd_params(x, weight, bias, out, silu, seq_idx=None, initial_states=None, final_states=None):
    p = FwdParams()
    p.batch, p.dim, p.seqlen = x.shape
    p.width = weight.shape[1]
    p.x_dtype, p.w_dtype, p.silu = DTYPES[x.dtype], DTYPES[weight.dtype], int(silu)
    _set3(p, "x", "x", x)
    p.weight, p.w_stride_c, p.w_stride_w = _ptr(weight), weight.stride(0), weight.stride(1)
    p.bias = _ptr(bias)
    _set3(p, "out", "out", out)
    p.seq_idx = _ptr(seq_idx)
    _set3(p, "init", "initial_states", initial_states)
    _set3(p, "final", "final_states", final_states)
    return p


def bwd_params(x, weight, bias, dout, dx, dweight, dbias, silu, seq_idx=None, initial_states=None,
               dfinal_states=None, dinitial_states=None):
    p = BwdParams()
    p.batch, p.dim, p.seqlen = x.shape
    p.width = weight.shape[1]
    p.x_dtype, p.w_dtype, p.silu = DTYPES[x.dtype], DTYPES[weight.dtype], int(silu)
    _set3(p, "x", "x", x)
    p.weight, p.w_stride_c, p.w_stride_w = _ptr(weight), weight.stride(0), weight.stride(1)
    p.bias = _ptr(bias)
    _set3(p, "dout", "dout", dout)
    p.seq_idx = _ptr(seq_idx)
    _set3(p, "init", "initial_states", initial_states)
    _set3(p, "dfinal", "dfinal_states", dfinal_states)
    _set3(p, "dx", "dx", dx)
    p.dweight, p.dw_stride_c, p.dw_stride_w = _ptr(dweight), dweight.stride(0), dweight.stride(1)
    p.dbias = _ptr(dbias)
    _set3(p, "dinit", "dinitial_states", dinitial_states)
    return p


def update_params(x, conv_state, weight, bias, out, silu, cache_seqlens=None, conv_state_indices=None):
    p = UpdateParams()
    p.batch, p.dim, p.seqlen = x.shape
    p.width = weight.shape[1]
    p.state_len, p.state_batch = conv_state.shape[2], conv_state.shape[0]
    p.x_dtype, p.w_dtype, p.silu = DTYPES[x.dtype], DTYPES[weight.dtype], int(silu)
    _set3(p, "x", "x", x)
    _set3(p, "state", "conv_state", conv_state)
    p.weight, p.w_stride_c, p.w_stride_w = _ptr(weight), weight.stride(0), weight.stride(1)
    p.bias = _ptr(bias)
    _set3(p, "out", "out", out)
    p.cache_seqlens, p.conv_state_indices = _ptr(cache_seqlens), _ptr(conv_state_indices)
    return p


def varlen_params(x, cu_seqlens, states):
    p = VarlenParams()
    p.batch, p.dim, p.state_len = states.shape
    p.x_dtype = DTYPES[x.dtype]
    p.cu_seqlens_is_int64 = int(cu_seqlens.dtype == torch.int64)
    p.total_tokens = x.shape[0]
    p.x, p.x_stride_t, p.x_stride_c = _ptr(x), x.stride(0), x.stride(1)
    p.cu_seqlens = _ptr(cu_seqlens)
    p.states = _ptr(states)
    p.states_stride_b, p.states_stride_c, p.states_stride_l = states.stride()
    return p


def declare(lib):
    """Attach argument/return types to the entry points of a loaded libcc1d.so."""
    lib.cc1d_strerror.restype = C.c_char_p
    lib.cc1d_strerror.argtypes = [C.c_int]
    for name, st in (("fwd", FwdParams), ("bwd", BwdParams), ("update", UpdateParams),
                     ("varlen_states", VarlenParams)):
        getattr(lib, "cc1d_validate_" + name).argtypes = [C.POINTER(st)]
    lib.cc1d_fwd.argtypes = [C.POINTER(FwdParams), vp]
    lib.cc1d_bwd_workspace_bytes.argtypes = [C.POINTER(BwdParams), C.POINTER(C.c_size_t)]
    lib.cc1d_bwd.argtypes = [C.POINTER(BwdParams), vp, C.c_size_t, vp]
    if hasattr(lib, "cc1d_bwd_noalloc"):
        lib.cc1d_bwd_noalloc.argtypes = [C.POINTER(BwdParams), vp]
    lib.cc1d_update.argtypes = [C.POINTER(UpdateParams), vp]
    lib.cc1d_varlen_states.argtypes = [C.POINTER(VarlenParams), vp]
    lib.cc1d_fwd_varlen_states.argtypes = [C.POINTER(FwdParams), C.POINTER(VarlenParams), vp]
    lib.cc1d_set_tunable.argtypes = [C.c_char_p, i32]
    lib.cc1d_get_tunable.argtypes = [C.c_char_p, C.POINTER(i32)]
    return lib
