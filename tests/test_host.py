"""CPU-only checks of the drop-in boundary: the C-ABI library loads and exports what the header
declares, argument checks fail loudly without touching a GPU, and the host-side mirror keeps the
reference's interface and error behaviour."""
import ctypes
import inspect
import os
import re

import pytest
import torch

from separableflowthesis_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "sepcorr.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sepcorr_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = header_symbols()
    assert len(names) == 44
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"libsepcorr.so does not export {n}"
    assert sorted(_lib.SIGNATURES) == names          # the ctypes table covers the header, nothing else


def test_abi_version_and_workspace_query():
    lib = _lib.load()
    assert lib.sepcorr_abi_version() == 2
    assert lib.sepcorr_backward_workspace_bytes(0, 1, 1, 1, 1, 1) == 0
    n = lib.sepcorr_backward_workspace_bytes(2, 55, 128, 55, 128, 256)
    # d_f2-sized partial buffers, then (C == 256) the transposed copy of up to 11 weight fields of size B*H2*N1,
    # then what the weight-gradient sweep of the compression backward can use (a forward-type sweep)
    part, fields = 2 * 55 * 128 * 256 * 4, 11 * 2 * 55 * (55 * 128) * 4
    fwd = lib.sepcorr_forward_workspace_bytes(2, 55, 128, 55, 128, 256, 8)
    assert fwd > 0 and fwd % 256 == 0
    # (kernels dealt out in pieces run one after the other and share the memory: the largest region counts)
    assert n >= max(fields, fwd, 2 * part) and n % 256 == 0
    # whole tiles fill the chip: nothing to gain from scratch (1020 tiles of 8 waves on 256 units)
    assert lib.sepcorr_forward_workspace_bytes(1, 136, 240, 136, 240, 256, 4) == 0
    assert lib.sepcorr_forward_workspace_bytes(0, 1, 1, 1, 1, 1, 2) == 0
    one = ctypes.c_void_p(256)
    args = (2, 55, 128, 55, 128, 256)
    assert lib.sepcorr_max_avg_forward(one, one, one, one, *args, one, 16, None) == -3          # too small
    assert lib.sepcorr_max_avg_forward(one, one, one, one, *args, ctypes.c_void_p(260), 1 << 40, None) == -3   # misaligned
    assert b"aligned" in lib.sepcorr_last_error()


def test_argument_checks_precede_any_launch():
    lib = _lib.load()
    one = ctypes.c_void_p(256)   # never dereferenced: every call below must fail in the checks
    assert lib.sepcorr_max_avg_forward(None, one, one, one, 1, 1, 1, 1, 1, 1, None, 0, None) == -1
    assert b"NULL" in lib.sepcorr_last_error()
    assert lib.sepcorr_max_avg_forward(one, one, one, one, 1, 1, 1, 1, 0, 1, None, 0, None) == -1
    assert lib.sepcorr_max_avg_forward(one, one, one, one, 1, 1, 1, 1, 2049, 1, None, 0, None) == -1
    assert b"W2=2049" in lib.sepcorr_last_error()
    assert lib.sepcorr_max_argmax_avg_forward(one, one, one, one, one, one, 1, 1, 1, 1, 1, 2000, None, 0, None) == -1
    assert lib.sepcorr_compression_forward(one, one, one, one, one, one, 1, 1, 1, 1, 1, 1, 9, None, 0, None) == -1
    assert b"K=9" in lib.sepcorr_last_error()
    assert lib.sepcorr_compression_forward(one, one, one, one, one, one, 1, 1, 1, 1, 1, 1, 0, None, 0, None) == -1
    # 2^31 elements
    assert lib.sepcorr_max_avg_forward(one, one, one, one, 64, 1024, 1024, 4, 4, 64, None, 0, None) == -1
    # workspace missing / too small
    args = (2, 55, 128, 55, 128, 256)
    assert lib.sepcorr_max_argmax_avg_backward(one, one, one, one, one, one, one, one, *args, None, 0, None) == -3
    assert lib.sepcorr_compression_backward(one, one, one, one, one, one, one, one, one, one, *args, 4, one, 16, None) == -3
    assert b"workspace" in lib.sepcorr_last_error()
    # the documented 256-byte alignment is enforced by every backward entry point
    big = 1 << 40
    for ptr in (16, 128, 256 + 64):
        assert lib.sepcorr_max_argmax_avg_backward(one, one, one, one, one, one, one, one, *args, ctypes.c_void_p(ptr), big, None) == -3
        assert b"256-byte aligned" in lib.sepcorr_last_error()
    assert lib.sepcorr_fused_backward(*([one] * 12), *args, 4, ctypes.c_void_p(48), big, None) == -3
    assert lib.sepcorr_compression_backward(*([one] * 10), *args, 4, ctypes.c_void_p(48), big, None) == -3


def test_lookup_argument_checks_precede_any_launch():
    lib = _lib.load()
    one = ctypes.c_void_p(256)
    lv = (ctypes.c_void_p * 2)(256, 256)
    hw = (ctypes.c_int * 2)(4, 2)
    f = lib.sepcorr_lookup_forward
    assert f(None, lv, hw, hw, one, one, 1, 4, 4, 8, 2, 4, 1.0, None) == -1 and b"NULL" in lib.sepcorr_last_error()
    assert f(one, lv, hw, hw, one, one, 1, 4, 4, 8, 2, 9, 1.0, None) == -1 and b"radius" in lib.sepcorr_last_error()
    assert f(one, lv, hw, hw, one, one, 1, 4, 4, 8, 9, 4, 1.0, None) == -1 and b"levels" in lib.sepcorr_last_error()
    assert f(one, lv, hw, hw, one, one, 1, 4, 4, 1025, 2, 4, 1.0, None) == -1
    assert f(one, (ctypes.c_void_p * 2)(256, None), hw, hw, one, one, 1, 4, 4, 8, 2, 4, 1.0, None) == -1
    assert f(one, lv, (ctypes.c_int * 2)(4, 0), hw, one, one, 1, 4, 4, 8, 2, 4, 1.0, None) == -1
    n = lib.sepcorr_lookup_backward_workspace_bytes(hw, hw, 1, 4, 4, 8, 2, 4)
    assert n > 0 and n % 256 == 0
    assert lib.sepcorr_lookup_backward_workspace_bytes(hw, hw, 1, 4, 4, 8, 2, 0) == 0
    b = lib.sepcorr_lookup_backward
    assert b(one, lv, hw, hw, one, one, one, lv, 1, 4, 4, 8, 2, 4, 1.0, None, 0, None) == -3
    assert b(one, lv, hw, hw, one, one, one, lv, 1, 4, 4, 8, 2, 4, 1.0, ctypes.c_void_p(257), n, None) == -1
    assert b"aligned" in lib.sepcorr_last_error()


def test_lookup1d_argument_checks_precede_any_launch():
    lib = _lib.load()
    one = ctypes.c_void_p(256)
    f, b = lib.sepcorr_lookup1d_forward, lib.sepcorr_lookup1d_backward
    assert f(None, one, one, 1, 1, 16, 4, 4, 0, 0, 4, 4, None) == -1 and b"NULL" in lib.sepcorr_last_error()
    assert f(one, one, one, 1, 1, 16, 4, 4, 2, 0, 4, 4, None) == -1 and b"coord_channel" in lib.sepcorr_last_error()
    assert f(one, one, one, 1, 1, 16, 4, 4, 0, 0, 9, 4, None) == -1 and b"levels" in lib.sepcorr_last_error()
    assert f(one, one, one, 1, 1, 4, 4, 4, 0, 0, 4, 4, None) == -1 and b"too short" in lib.sepcorr_last_error()
    assert f(one, one, one, 1, 1, 16, 4, 4, 0, 0, 4, 17, None) == -1 and b"radius" in lib.sepcorr_last_error()
    assert f(one, one, one, 64, 64, 1024, 64, 64, 0, 0, 4, 4, None) == -1 and b"2^31" in lib.sepcorr_last_error()
    assert b(one, None, one, 1, 1, 16, 4, 4, 0, 0, 4, 4, None) == -1 and b"NULL" in lib.sepcorr_last_error()


def test_cpu_tensors_are_refused_like_check_cuda():
    from separableflowthesis_amd import MemorySaver
    f = torch.randn(1, 2, 2, 4)
    for call in (lambda: MemorySaver.max_avg_forward(f, f),
                 lambda: MemorySaver.max_argmax_avg_forward(f, f),
                 lambda: MemorySaver.compression_forward(f, f, f, f),
                 lambda: MemorySaver.compression_backward(f, f, f, f, f, f),
                 lambda: MemorySaver.max_argmax_avg_backward(f, f, f, f, f, f)):
        with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
            call()


def test_native_module_mirrors_the_five_reference_functions():
    from separableflowthesis_amd import MemorySaver
    expect = {
        "max_avg_forward": ["img1_features_l0", "img2_features_lk"],
        "max_argmax_avg_forward": ["img1_features_l0", "img2_features_lk"],
        "max_argmax_avg_backward": ["img1_features_l0", "img2_features_lk", "argmax_output_u", "argmax_output_v",
                                    "grad_MaxAvg_u", "grad_MaxAvg_v"],
        "compression_forward": ["img1_features_l0", "img2_features_lk", "attention_weights_u", "attention_weights_v"],
        "compression_backward": ["img1_features_l0", "img2_features_lk", "attention_weights_u", "attention_weights_v",
                                 "grad_compressed_output_u", "grad_compressed_output_v"],
    }
    for name, params in expect.items():
        assert list(inspect.signature(getattr(MemorySaver, name)).parameters) == params


def test_autograd_function_interface():
    import separableflowthesis_amd as pkg
    for cls, nin in ((pkg.ComputeMaxAvgFunction, 2), (pkg.ComputeMaxArgmaxAvgFunction, 2),
                     (pkg.ComputeSelfCompressionFunction, 4)):
        assert issubclass(cls, torch.autograd.Function)
        assert len(inspect.signature(cls.forward).parameters) == nin + 1
    with pytest.raises(NotImplementedError):
        pkg.ComputeMaxAvgFunction.backward(None, None, None)
    f = torch.randn(1, 2, 2, 4)
    with pytest.raises(AssertionError):
        pkg.ComputeMaxAvgFunction.apply(f.permute(0, 2, 1, 3), f)


def test_corr_block_guards_and_pyramid():
    from separableflowthesis_amd import AlternateCorrBlockSepflow
    fmap = torch.randn(1, 8, 11, 13)
    with pytest.raises(Exception, match="NLF"):
        AlternateCorrBlockSepflow(fmap, fmap, guid=torch.zeros(1))
    blk = AlternateCorrBlockSepflow(fmap, fmap, None, num_levels=4, support_backward=True)
    assert [tuple(p.shape[2:]) for p in blk.pyramid] == [(11, 13), (5, 6), (2, 3), (1, 1)]
    assert blk.max_avg_function.__name__ == "ComputeMaxArgmaxAvgFunction"
    assert AlternateCorrBlockSepflow(fmap, fmap, None).max_avg_function.__name__ == "ComputeMaxAvgFunction"
    # the lookup is native as well (the reference raises NotImplementedError here, core/corr.py:491-492):
    # CPU tensors are refused, there is no fallback
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        blk(torch.zeros(1, 2, 11, 13))


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libsepcorr.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load()
