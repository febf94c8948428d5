"""Runs the host-buffer test cases of ukref.py through the device library's
C ABI: upload, call iree_amd_uk_*_p with device pointers, download."""
import ctypes as C

import numpy as np
import torch

import iree_amd


def _to_dev(a):
    t = torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy())
    return t.cuda()


def _check(st):
    if st != 0:
        raise iree_amd.UkError(st, iree_amd.load_library().iree_amd_uk_last_error().decode())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def run_mmt4d(case, flags=None):
    lib = iree_amd.load_library()
    lhs, rhs, out = _to_dev(case.lhs), _to_dev(case.rhs), _to_dev(case.out_init)
    p = case.params(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), flags=flags)
    _check(lib.iree_amd_uk_mmt4d_p(C.byref(p), _stream()))
    torch.cuda.synchronize()
    return out.cpu().numpy().view(case.out_init.dtype)


def run_batch_mmt4d(case):
    lib = iree_amd.load_library()
    lhs, rhs, out = _to_dev(case.lhs), _to_dev(case.rhs), _to_dev(case.out_init)
    p = case.params(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr())
    _check(lib.iree_amd_uk_batch_mmt4d(C.byref(p), case.batch, case.lhs_batch_stride,
                                       case.rhs_batch_stride, case.out_batch_stride, _stream()))
    torch.cuda.synchronize()
    return out.cpu().numpy().view(case.out_init.dtype)


def run_pack(case):
    lib = iree_amd.load_library()
    inp, out = _to_dev(case.inp), _to_dev(case.out_init)
    p = case.params(inp.data_ptr(), out.data_ptr())
    _check(lib.iree_amd_uk_pack_p(C.byref(p), _stream()))
    torch.cuda.synchronize()
    return out.cpu().numpy().view(case.out_init.dtype)


def run_unpack(case):
    lib = iree_amd.load_library()
    inp, out = _to_dev(case.inp), _to_dev(case.out_init)
    p = case.params(inp.data_ptr(), out.data_ptr())
    _check(lib.iree_amd_uk_unpack_p(C.byref(p), _stream()))
    torch.cuda.synchronize()
    return out.cpu().numpy().view(case.out_init.dtype)
