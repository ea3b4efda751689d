"""Host-only checks of the C ABI (no GPU, no kernel launch): the library loads, exports
every function include/cc1d.h declares, the ctypes mirror has the header's struct sizes,
and every validation path returns the documented status.  The validation codes restate
the TORCH_CHECKs of the reference binding (csrc/causal_conv1d.cpp:158-199, 273-327,
475-542)."""
import ctypes as C
import os
import re
import subprocess
import tempfile

import pytest
import torch

import cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "cc1d.h")

OK, E_NULL, E_DTYPE, E_WIDTH, E_SHAPE, E_XLAYOUT, E_C8, E_S8, E_ALIGN, E_SEQ_LAYOUT = range(0, -10, -1)
E_OUT_LAYOUT, E_STATE_LAYOUT, E_STATE_LEN, E_WS, E_BIAS, E_SEQ_STATES = range(-10, -16, -1)


@pytest.fixture(scope="module")
def lib(cc1d_lib):
    return cabi.declare(cc1d_lib)


def test_every_declared_symbol_is_exported(lib):
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(cc1d_[a-z_0-9]+)\s*\(", text)
    assert len(set(names)) >= 15 and {'cc1d_fwd', 'cc1d_bwd', 'cc1d_update', 'cc1d_varlen_states'} <= set(names)
    for n in set(names):
        assert hasattr(lib, n), f"{n} declared in cc1d.h but not exported"
    assert lib.cc1d_abi_version() == 1


def test_struct_sizes_match_the_header():
    src = '#include <stdio.h>\n#include "cc1d.h"\nint main(void){printf("%zu %zu %zu %zu\\n",' \
          'sizeof(cc1d_fwd_params),sizeof(cc1d_bwd_params),sizeof(cc1d_update_params),sizeof(cc1d_varlen_params));return 0;}'
    with tempfile.TemporaryDirectory() as d:
        open(os.path.join(d, "s.c"), "w").write(src)
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.dirname(HEADER),
                        os.path.join(d, "s.c"), "-o", os.path.join(d, "s")], check=True)
        sizes = [int(v) for v in subprocess.run([os.path.join(d, "s")], capture_output=True, text=True).stdout.split()]
    assert sizes == [C.sizeof(cabi.FwdParams), C.sizeof(cabi.BwdParams),
                     C.sizeof(cabi.UpdateParams), C.sizeof(cabi.VarlenParams)]


def test_strerror_texts(lib):
    assert lib.cc1d_strerror(0) == b"success"
    assert b"width between 2 and 4" in lib.cc1d_strerror(E_WIDTH)
    assert b"divisible by 8" in lib.cc1d_strerror(E_C8)
    assert b"multiples of 8" in lib.cc1d_strerror(E_S8)
    assert b"channel last" in lib.cc1d_strerror(E_SEQ_LAYOUT)
    assert b"unknown" in lib.cc1d_strerror(-999)


def _fwd(B=2, D=16, L=24, W=4, channel_last=False, dtype=torch.float32):
    x = torch.zeros(B, L, D, dtype=dtype).transpose(1, 2) if channel_last else torch.zeros(B, D, L, dtype=dtype)
    w, b = torch.zeros(D, W), torch.zeros(D)
    out = torch.empty_like(x)
    keep = (x, w, b, out)
    return cabi.fwd_params(x, w, b, out, True), keep


def test_validate_fwd_paths(lib):
    v = lib.cc1d_validate_fwd
    assert v(None) == E_NULL
    p, _k = _fwd()
    assert v(p) == OK
    p, _k = _fwd(channel_last=True)
    assert v(p) == OK
    p, _k = _fwd(); p.width = 5
    assert v(p) == E_WIDTH
    p, _k = _fwd(); p.width = 1
    assert v(p) == E_WIDTH
    p, _k = _fwd(); p.x_dtype = 7
    assert v(p) == E_DTYPE
    p, _k = _fwd(); p.seqlen = -1
    assert v(p) == E_SHAPE
    p, _k = _fwd(); p.out = None
    assert v(p) == E_NULL
    p, _k = _fwd(); p.x_stride_c, p.x_stride_l = 48, 2
    assert v(p) == E_XLAYOUT
    p, _k = _fwd(D=12, channel_last=True)
    assert v(p) == E_C8
    p, _k = _fwd(channel_last=True); p.x_stride_l = 20
    assert v(p) == E_S8
    p, _k = _fwd(channel_last=True); p.x = p.x + 4
    assert v(p) == E_ALIGN
    p, _k = _fwd(channel_last=True); p.out_stride_c, p.out_stride_l = 24, 1
    assert v(p) == E_OUT_LAYOUT
    p, _k = _fwd(); p.out_stride_l = 2
    assert v(p) == E_OUT_LAYOUT
    seq = torch.zeros(2, 24, dtype=torch.int32)
    p, _k = _fwd(); p.seq_idx = seq.data_ptr()
    assert v(p) == E_SEQ_LAYOUT
    p, _k = _fwd(channel_last=True); p.seq_idx = seq.data_ptr()
    assert v(p) == OK
    p, _k = _fwd(); p.batch = 0; p.x = None
    assert v(p) == OK and lib.cc1d_fwd(p, None) == OK      # empty problem: nothing to launch


def test_validate_fwd_states_that_share_memory(lib):
    """initial_states and final_states may be one tensor (same address, same strides); two
    different views are accepted when they share no element and refused when they do."""
    v = lib.cc1d_validate_fwd
    B, D, W = 2, 16, 4

    def with_states(init, fin):
        p, keep = _fwd(B=B, D=D, W=W, channel_last=True)
        cabi._set3(p, "init", "initial_states", init)
        cabi._set3(p, "final", "final_states", fin)
        return p, (keep, init, fin)

    state = torch.zeros(B, W - 1, D).transpose(1, 2)
    p, _k = with_states(state, state)
    assert v(p) == OK                                   # one buffer
    p, _k = with_states(state, torch.zeros(B, W - 1, D).transpose(1, 2))
    assert v(p) == OK                                   # two allocations
    big = torch.zeros(B, 8, D).transpose(1, 2)          # (B, D, 8): two windows of one cache
    p, _k = with_states(big[:, :, 0:3], big[:, :, 3:6])
    assert v(p) == OK                                   # interleaved in memory, no element in common
    p, _k = with_states(big[:, :, 0:3], big[:, :, 2:5])
    assert v(p) == E_STATE_LAYOUT                       # share position 2
    p, _k = with_states(big[:, :, 2:5], big[:, :, 0:3])
    assert v(p) == E_STATE_LAYOUT
    p, _k = with_states(state, state.contiguous().transpose(1, 2)[:, :W - 1, :W - 1].new_zeros(B, D, W - 1))
    assert v(p) == OK
    flat = torch.zeros(B * D * (W - 1))
    a = flat.as_strided((B, D, W - 1), (D * (W - 1), 1, D))          # dim fastest
    c = flat.as_strided((B, D, W - 1), (D * (W - 1), W - 1, 1))      # seqlen fastest, same memory
    p, _k = with_states(a, c)
    assert v(p) == E_STATE_LAYOUT                       # same bytes under two different views


def test_outputs_that_share_elements_with_inputs_are_refused(lib):
    """No kernel works in place (a row's halo is read by another wavefront than the one that
    writes the positions in front of it).  Refused only where a shared element is certain: the
    same nested strides for both views.  Views that merely interleave in memory pass."""
    E_IN_PLACE = -20
    B, D, L, W = 2, 16, 24, 4
    w, b = torch.zeros(D, W), torch.zeros(D)

    def fwd(x, out):
        return lib.cc1d_validate_fwd(cabi.fwd_params(x, w, b, out, True))

    for channel_last in (False, True):
        wide = torch.zeros(B, L, 3 * D).transpose(1, 2) if channel_last else torch.zeros(B, 3 * D, L)
        x = wide[:, 0:D, :]
        assert fwd(x, x) == E_IN_PLACE                             # in place
        assert fwd(x, wide[:, D:2 * D, :]) == OK                   # a neighbouring slice of the same buffer
        assert fwd(x, wide[:, D // 2:D // 2 + D, :]) == E_IN_PLACE  # half of the channels in common
        assert fwd(wide[:, D:2 * D, :], x) == OK
        assert fwd(wide[:, D // 2:D // 2 + D, :], x) == E_IN_PLACE
        long_ = torch.zeros(B, 2 * L + 8, D).transpose(1, 2) if channel_last else torch.zeros(B, D, 2 * L + 8)
        assert fwd(long_[:, :, 0:L], long_[:, :, L:2 * L]) == OK   # two windows along seqlen
        assert fwd(long_[:, :, 0:L], long_[:, :, L - 1:2 * L - 1]) == E_IN_PLACE
        assert fwd(long_[:, :, 8:L + 8], long_[:, :, 0:L]) == E_IN_PLACE
        fresh = torch.zeros_like(wide)[:, 0:D, :]
        assert fwd(x, fresh) == OK
    p, _k = _bwd(channel_last=True)
    assert lib.cc1d_validate_bwd(p) == OK
    p.dx, p.dx_stride_b, p.dx_stride_c, p.dx_stride_l = p.dout, p.dout_stride_b, p.dout_stride_c, p.dout_stride_l
    assert lib.cc1d_validate_bwd(p) == E_IN_PLACE                  # dx written over dout
    p, _k = _bwd(channel_last=False)
    p.dx, p.dx_stride_b, p.dx_stride_c, p.dx_stride_l = p.x, p.x_stride_b, p.x_stride_c, p.x_stride_l
    assert lib.cc1d_validate_bwd(p) == E_IN_PLACE                  # dx written over x
    assert b"in place" in lib.cc1d_strerror(E_IN_PLACE)


def _bwd(channel_last=False, bias=True):
    B, D, L, W = 2, 16, 24, 4
    mk = (lambda: torch.zeros(B, L, D).transpose(1, 2)) if channel_last else (lambda: torch.zeros(B, D, L))
    x, dout, dx = mk(), mk(), mk()
    w, b = torch.zeros(D, W), (torch.zeros(D) if bias else None)
    dw, db = torch.zeros(D, W), (torch.zeros(D) if bias else None)
    keep = (x, dout, dx, w, b, dw, db)
    return cabi.bwd_params(x, w, b, dout, dx, dw, db, True), keep


def test_validate_bwd_paths(lib):
    v = lib.cc1d_validate_bwd
    for cl in (False, True):
        p, _k = _bwd(cl)
        assert v(p) == OK
        n = C.c_size_t(123)
        assert lib.cc1d_bwd_workspace_bytes(p, C.byref(n)) == OK
        assert n.value % 16 == 0
        if cl:
            assert n.value > 0
            assert lib.cc1d_bwd(p, None, 0, None) == E_WS        # rejected before any launch
    p, _k = _bwd(); p.dbias = None
    assert v(p) == E_BIAS
    p, _k = _bwd(); p.dweight = None
    assert v(p) == E_NULL
    p, _k = _bwd(True); p.dout_stride_c, p.dout_stride_l = 24, 1
    assert v(p) == E_OUT_LAYOUT
    p, _k = _bwd(True); p.dx_stride_l = 12
    assert v(p) == E_S8
    seq = torch.zeros(2, 24, dtype=torch.int32)
    p, _k = _bwd(False); p.seq_idx = seq.data_ptr()
    assert v(p) == E_SEQ_LAYOUT
    st = torch.zeros(2, 3, 16).transpose(1, 2)
    p, _k = _bwd(True); p.seq_idx = seq.data_ptr(); p.initial_states = st.data_ptr()
    assert v(p) == E_SEQ_STATES
    assert lib.cc1d_bwd_workspace_bytes(p, None) == E_NULL


def test_validate_update_and_varlen_paths(lib):
    x, st = torch.zeros(4, 16, 1), torch.zeros(4, 16, 3)
    w, b, out = torch.zeros(16, 4), torch.zeros(16), torch.zeros(4, 16, 1)
    v = lib.cc1d_validate_update
    assert v(cabi.update_params(x, st, w, b, out, True)) == OK
    p = cabi.update_params(x, torch.zeros(4, 16, 2), w, b, out, True)
    assert v(p) == E_STATE_LEN
    p = cabi.update_params(x, torch.zeros(9, 16, 3), w, b, out, True)
    assert v(p) == E_SHAPE                                    # bigger state needs conv_state_indices
    idx = torch.zeros(4, dtype=torch.int32)
    p = cabi.update_params(x, torch.zeros(9, 16, 3), w, b, out, True, conv_state_indices=idx)
    assert v(p) == OK
    p = cabi.update_params(x, st, w, b, out, True); p.conv_state = None
    assert v(p) == E_NULL
    assert v(None) == E_NULL

    xs, cu, states = torch.zeros(10, 16), torch.tensor([0, 4, 10], dtype=torch.int32), torch.zeros(2, 16, 3)
    vv = lib.cc1d_validate_varlen_states
    assert vv(cabi.varlen_params(xs, cu, states)) == OK
    p = cabi.varlen_params(xs, cu, states); p.cu_seqlens = None
    assert vv(p) == E_NULL
    p = cabi.varlen_params(xs, cu, states); p.x_dtype = 9
    assert vv(p) == E_DTYPE
    p = cabi.varlen_params(xs, cu, states); p.total_tokens = -1
    assert vv(p) == E_SHAPE
    assert vv(None) == E_NULL


def test_tunables_round_trip(lib):
    val = C.c_int32(-1)
    assert lib.cc1d_get_tunable(b"fwd_cl_rows", C.byref(val)) == OK and val.value == 0
    assert lib.cc1d_set_tunable(b"fwd_cl_rows", 64) == OK
    assert lib.cc1d_get_tunable(b"fwd_cl_rows", C.byref(val)) == OK and val.value == 64
    assert lib.cc1d_set_tunable(b"fwd_cl_rows", 0) == OK
    assert lib.cc1d_set_tunable(b"no_such_knob", 1) == -18
    assert lib.cc1d_set_tunable(None, 1) == E_NULL
