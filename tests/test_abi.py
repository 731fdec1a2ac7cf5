"""The C-ABI library loads, exports every symbol include/mpsa.h declares, and rejects bad arguments on the
host (no kernel is launched; runs without a GPU)."""
import ctypes
import os
import re

import pytest
import torch

from conftest import ROOT
from ours import _lib


def _declared():
    text = open(os.path.join(ROOT, "include", "mpsa.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mpsa_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared()
    assert "mpsa_attn_fwd" in names and "mpsa_quantize_mx" in names and len(names) >= 11
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), f"{n} declared in mpsa.h but not exported"
    assert sorted(_lib.SIGNATURES) == names
    assert _lib.lib().mpsa_version() >= 100


def test_host_side_argument_validation():
    L = _lib.lib()
    null = ctypes.c_void_p(0)
    one = ctypes.c_void_p(16)           # never dereferenced: validation fails first
    st = (ctypes.c_int64 * 4)(1, 1, 32, 1)
    assert L.mpsa_quantize_mx(null, 0, 1, 1, 1, 32, st, null, 1.0, 4, 3, one, one, 1, null) == -1
    assert b"null" in L.mpsa_last_error()
    st_ok = (ctypes.c_int64 * 4)(64, 64, 64, 1)
    assert L.mpsa_quantize_mx(one, 0, 1, 1, 1, 48, st_ok, null, 1.0, 4, 3, one, one, 1, null) == -1      # D % 32
    assert L.mpsa_quantize_mx(one, 2, 1, 1, 1, 64, st_ok, null, 1.0, 4, 3, one, one, 1, null) == -1      # f32 input
    assert L.mpsa_quantize_mx(one, 0, 1, 1, 1, 64, st_ok, null, 1.0, 9, 3, one, one, 1, null) == -1      # bad format
    assert L.mpsa_quantize_mx(one, 0, 1, 1, 2, 64, st_ok, null, 1.0, 4, 3, one, one, 1, null) == -1      # out_rows < N
    assert L.mpsa_quantize_mx(ctypes.c_void_p(24), 0, 1, 1, 1, 64, st_ok, null, 1.0, 4, 3, one, one, 1, null) == -2
    assert L.mpsa_quantize_mx(one, 0, 1, 1, 1, 64, st_ok, ctypes.c_void_p(8), 1.0, 4, 3, one, one, 1, null) == -2   # sub alignment
    assert L.mpsa_seq_mean_workspace(2, 3, 1000, 64) == 2 * 3 * 4 * 64 * 4
    assert L.mpsa_seq_mean(one, 0, 1, 1, 8, 64, st_ok, null, one, null) == -1                      # no workspace
    assert L.mpsa_seq_mean(one, 0, 1, 1, 8, 96, st_ok, one, one, null) == -3                       # D = 96
    assert L.mpsa_gemm_mx(one, one, 4, one, one, 4, 100, 256, 96, one, 0, 256, null) == -3         # K % 64
    assert L.mpsa_gemm_mx(one, one, 4, one, one, 4, 256, 256, 128, one, 7, 256, null) == -1        # bad dtype
    assert L.mpsa_gemm_mx(one, one, 4, one, one, 3, 256, 256, 128, one, 0, 256, null) == -1        # bad format of B
    assert L.mpsa_gemm_mx_packed(one, one, 4, one, one, 4, 100, 256, 128, one, 0, 256, null) == -3  # packed: M % 128
    assert L.mpsa_fp8_encode(null, 4, 0, one, null) == -1
    assert L.mpsa_fp8_encode(one, 4, 4, one, null) == -1                                           # E2M1 is not an FP8 format
    assert L.mpsa_seq_mean_static(one, 0, 1, 64, 262144, 128, st_ok, one, null) == -3              # beyond the built-in array
    assert L.mpsa_v_tiles(one, 0, 1, 1, 128, 96, st_ok, 128, one, null) == -3                      # D = 96
    so = (ctypes.c_int64 * 4)(128 * 128, 128 * 128, 128, 1)
    args = [one] * 8 + [0, one, 0, one, 0, so, 1, 4, 3, 128, 128, 128, 128, 1, 2, null]
    assert L.mpsa_attn_fwd(*args) == -1                                                            # Hq % Hkv
    args = [null] * 4 + [one] * 4 + [0, one, 0, one, 0, so, 1, 4, 2, 128, 128, 128, 128, 1, 2, null]
    assert L.mpsa_attn_fwd(*args) == -1                                                            # diag needs 4-bit Q
    args = [one] * 8 + [0, one, 0, one, 0, so, 1, 4, 2, 128, 128, 96, 128, 1, 2, null]
    assert L.mpsa_attn_fwd(*args) == -3                                                            # D = 96
    args = [one] * 8 + [0, one, 0, one, 0, so, 1, 4, 2, 128, 256, 128, 128, 1, 0, null]
    assert L.mpsa_attn_fwd(*args) == -1                                                            # causal with nq != nk
    # tile skipping ahead of the attention kernel: the shapes it takes, the operands a mode multiplies, the lists' memory
    assert L.mpsa_skip_route_supported(8192, 8192, 128, 128, 1, 2) == 1 and L.mpsa_skip_route_supported(8192, 8192, 64, 128, 1, 2) == 0
    assert L.mpsa_skip_route_supported(8192, 8192, 128, 128, 1, 4) == 0                            # the mixed type
    assert L.mpsa_skip_route_supported(300, 77, 128, 128, 0, 0) == 1 and L.mpsa_skip_route_supported(300, 77, 128, 128, 0, 2) == 0
    assert L.mpsa_skip_route_supported(128 * 2049, 128 * 2049, 128, 128, 1, 0) == 0                # more key tiles than its LDS holds
    assert L.mpsa_skip_route_workspace(1, 4, 1000, 300, 128) == 4 * 8 * 3 * 4
    shape = [0, 1, 4, 2, 1024, 1024, 128, 128, 1]
    assert L.mpsa_skip_route(*([one] * 8 + shape + [4, 1.0, one, null, one, one, null, null])) == -3          # mixed
    assert L.mpsa_skip_route(*([one, one, null, null] + [one] * 4 + shape + [2, 1.0, one, null, one, one, null, null])) == -1   # diag without 8-bit Q
    assert L.mpsa_skip_route(*([one] * 8 + shape + [2, float("nan"), one, null, one, one, null, null])) == -1
    assert L.mpsa_skip_route(*([one] * 8 + shape + [2, 1.0, null, null, one, one, null, null])) == -1           # no workspace
    assert L.mpsa_skip_route(*([one] * 8 + shape + [2, 1.0, one, null, ctypes.c_void_p(18), one, null, null])) == -2   # order misaligned
    so2 = (ctypes.c_int64 * 4)(128 * 128, 128 * 128, 128, 1)
    routed = [one, one, null, one] + [one] * 4 + [0, one, 0, one, 0, so2, 1, 4, 2, 128, 128, 128, 128, 1, one, one, null]
    assert L.mpsa_attn_fwd_routed(*routed) == -1 and b"whole" in L.mpsa_last_error()               # half an operand set
    assert L.mpsa_e2m1_pack(null, 2, 3, 4, one, null) == -1                                         # null input
    assert L.mpsa_e2m1_pack(null, 0, 3, 4, null, null) == 0                                         # empty is fine
    assert L.mpsa_e2m1_encode(null, 4, one, null) == -1
    assert L.mpsa_e2m1_encode(null, 0, null, null) == 0                                            # empty is fine


def test_python_entry_points_refuse_cpu_tensors_and_bad_arguments():
    from ours.mxfp import MXFP4Tensor, MXScaleTensor
    from ours.mxfp_attn import mxfp_attn
    from ours.mxfp_attn_kernel import mxfp_attn_kernel
    from ours.block_scaled_matmul import block_scaled_matmul, make_configs
    x = torch.zeros(1, 2, 128, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        mxfp_attn(x, x, x)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        MXFP4Tensor(data=torch.zeros(4))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        MXScaleTensor(data=torch.ones(4))
    with pytest.raises(AssertionError, match="seq_len"):
        mxfp_attn(x[:, :, :64], x[:, :, :64], x[:, :, :64])
    with pytest.raises(AssertionError, match="headdim"):
        mxfp_attn(torch.zeros(1, 2, 128, 96), torch.zeros(1, 2, 128, 96), torch.zeros(1, 2, 128, 96))
    with pytest.raises(ValueError):
        MXFP4Tensor()
    with pytest.raises(ValueError, match="Unsupported dtype"):
        block_scaled_matmul(x, x, x, x, torch.int8, 256, 256, 128, make_configs("mxfp4"))
    with pytest.raises(ValueError, match="Invalid block scale type"):
        make_configs("nvfp4")
    assert make_configs("mixed")["ELEM_PER_BYTE_A"] == 1 and make_configs("mixed")["ELEM_PER_BYTE_B"] == 2
    t = MXFP4Tensor(data=torch.arange(16, dtype=torch.uint8).reshape(2, 8), dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="no CPU"):
        t.to_packed_tensor(dim=1)
