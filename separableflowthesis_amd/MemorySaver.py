"""Python face of the native module the reference calls `MemorySaver`.

Same five functions, argument order and return lists as the reference's pybind module
(libs/MemorySaver/src/MemorySaver_cuda.cpp:105-112), taking torch tensors.  torch is used for
device memory and the current stream only; the arithmetic happens in libsepcorr.so.

Checks mirror CHECK_CUDA / CHECK_CONTIGUOUS (MemorySaver_cuda.cpp:6-8) and add the dtype and
shape agreement the reference leaves unchecked; every violation raises RuntimeError.
"""
import torch

from . import _lib


def _check(name, t, dtype=torch.float32, ndim=None):
    if not isinstance(t, torch.Tensor):
        raise RuntimeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if t.dtype != dtype:
        raise RuntimeError(f"{name} must have dtype {dtype}, got {t.dtype}")
    if ndim is not None and t.dim() != ndim:
        raise RuntimeError(f"{name} must have {ndim} dimensions, got {t.dim()}")


def _dims(f1, f2):
    _check("img1_features_l0", f1, ndim=4)
    _check("img2_features_lk", f2, ndim=4)
    if f1.device != f2.device:
        raise RuntimeError("img1_features_l0 and img2_features_lk must be on the same device")
    B, H1, W1, C = f1.shape
    B2, H2, W2, C2 = f2.shape
    if B != B2 or C != C2:
        raise RuntimeError(f"batch/feature sizes differ: {tuple(f1.shape)} vs {tuple(f2.shape)}")
    return B, H1, W1, H2, W2, C


def _expect(name, t, shape, device, dtype=torch.float32):
    _check(name, t, dtype=dtype, ndim=len(shape))
    if tuple(t.shape) != tuple(shape):
        raise RuntimeError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    if t.device != device:
        raise RuntimeError(f"{name} must be on {device}")


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _workspace(lib, dims, device):
    n = lib.sepcorr_backward_workspace_bytes(*dims)
    ws = torch.empty(max(n, 1), dtype=torch.uint8, device=device)
    return ws, n


def _fwd_workspace(lib, dims, K, device):
    """Optional scratch of the forward-type sweeps (lets them use the whole chip when tiles do not divide evenly)."""
    n = lib.sepcorr_forward_workspace_bytes(*dims, K)
    if n == 0:
        return None, None, 0
    ws = torch.empty(n, dtype=torch.uint8, device=device)
    return ws, ws.data_ptr(), n


def max_avg_forward(img1_features_l0, img2_features_lk):
    """-> [max_avg_output_u (B,H1,W1,2,H2), max_avg_output_v (B,H1,W1,2,W2)]"""
    f1, f2 = img1_features_l0, img2_features_lk
    B, H1, W1, H2, W2, C = _dims(f1, f2)
    lib = _lib.load()
    with torch.cuda.device(f1.device):
        out_u = torch.empty((B, H1, W1, 2, H2), dtype=f1.dtype, device=f1.device)
        out_v = torch.empty((B, H1, W1, 2, W2), dtype=f1.dtype, device=f1.device)
        ws, wptr, n = _fwd_workspace(lib, (B, H1, W1, H2, W2, C), 2, f1.device)
        _lib.check(lib.sepcorr_max_avg_forward(f1.data_ptr(), f2.data_ptr(), out_u.data_ptr(), out_v.data_ptr(),
                                               B, H1, W1, H2, W2, C, wptr, n, _stream()))
    return [out_u, out_v]


def max_argmax_avg_forward(img1_features_l0, img2_features_lk):
    """-> [max_avg_output_u, max_avg_output_v, argmax_output_u (B,H1,W1,1,H2) i32, argmax_output_v (B,H1,W1,1,W2) i32]"""
    f1, f2 = img1_features_l0, img2_features_lk
    B, H1, W1, H2, W2, C = _dims(f1, f2)
    lib = _lib.load()
    with torch.cuda.device(f1.device):
        out_u = torch.empty((B, H1, W1, 2, H2), dtype=f1.dtype, device=f1.device)
        out_v = torch.empty((B, H1, W1, 2, W2), dtype=f1.dtype, device=f1.device)
        am_u = torch.empty((B, H1, W1, 1, H2), dtype=torch.int32, device=f1.device)
        am_v = torch.empty((B, H1, W1, 1, W2), dtype=torch.int32, device=f1.device)
        ws, wptr, n = _fwd_workspace(lib, (B, H1, W1, H2, W2, C), 2, f1.device)
        _lib.check(lib.sepcorr_max_argmax_avg_forward(f1.data_ptr(), f2.data_ptr(), out_u.data_ptr(), out_v.data_ptr(),
                                                      am_u.data_ptr(), am_v.data_ptr(), B, H1, W1, H2, W2, C, wptr, n,
                                                      _stream()))
    return [out_u, out_v, am_u, am_v]


def max_argmax_avg_backward(img1_features_l0, img2_features_lk, argmax_output_u, argmax_output_v,
                            grad_MaxAvg_u, grad_MaxAvg_v):
    """-> [grad_fmap1_l0 (B,H1,W1,C), grad_fmap2_lk (B,H2,W2,C)]"""
    f1, f2 = img1_features_l0, img2_features_lk
    B, H1, W1, H2, W2, C = _dims(f1, f2)
    dev = f1.device
    _expect("argmax_output_u", argmax_output_u, (B, H1, W1, 1, H2), dev, torch.int32)
    _expect("argmax_output_v", argmax_output_v, (B, H1, W1, 1, W2), dev, torch.int32)
    _expect("grad_MaxAvg_u", grad_MaxAvg_u, (B, H1, W1, 2, H2), dev)
    _expect("grad_MaxAvg_v", grad_MaxAvg_v, (B, H1, W1, 2, W2), dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        d1 = torch.empty_like(f1)
        d2 = torch.empty_like(f2)
        ws, n = _workspace(lib, (B, H1, W1, H2, W2, C), dev)
        _lib.check(lib.sepcorr_max_argmax_avg_backward(
            f1.data_ptr(), f2.data_ptr(), argmax_output_u.data_ptr(), argmax_output_v.data_ptr(),
            grad_MaxAvg_u.data_ptr(), grad_MaxAvg_v.data_ptr(), d1.data_ptr(), d2.data_ptr(),
            B, H1, W1, H2, W2, C, ws.data_ptr(), n, _stream()))
    return [d1, d2]


def compression_forward(img1_features_l0, img2_features_lk, attention_weights_u, attention_weights_v):
    """-> [compression_output_u (B,H1,W1,K,H2), compression_output_v (B,H1,W1,K,W2)]"""
    f1, f2 = img1_features_l0, img2_features_lk
    B, H1, W1, H2, W2, C = _dims(f1, f2)
    dev = f1.device
    _check("attention_weights_u", attention_weights_u, ndim=5)
    K = attention_weights_u.shape[3]
    _expect("attention_weights_u", attention_weights_u, (B, H1, W1, K, W2), dev)
    _expect("attention_weights_v", attention_weights_v, (B, H1, W1, K, H2), dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        cu = torch.empty((B, H1, W1, K, H2), dtype=f1.dtype, device=dev)
        cv = torch.empty((B, H1, W1, K, W2), dtype=f1.dtype, device=dev)
        ws, wptr, n = _fwd_workspace(lib, (B, H1, W1, H2, W2, C), K, dev)
        _lib.check(lib.sepcorr_compression_forward(
            f1.data_ptr(), f2.data_ptr(), attention_weights_u.data_ptr(), attention_weights_v.data_ptr(),
            cu.data_ptr(), cv.data_ptr(), B, H1, W1, H2, W2, C, K, wptr, n, _stream()))
    return [cu, cv]


def compression_backward(img1_features_l0, img2_features_lk, attention_weights_u, attention_weights_v,
                         grad_compressed_output_u, grad_compressed_output_v):
    """-> [grad_fmap1_l0, grad_fmap2_lk, grad_attention_u (B,H1,W1,K,W2), grad_attention_v (B,H1,W1,K,H2)]"""
    f1, f2 = img1_features_l0, img2_features_lk
    B, H1, W1, H2, W2, C = _dims(f1, f2)
    dev = f1.device
    _check("attention_weights_u", attention_weights_u, ndim=5)
    K = attention_weights_u.shape[3]
    _expect("attention_weights_u", attention_weights_u, (B, H1, W1, K, W2), dev)
    _expect("attention_weights_v", attention_weights_v, (B, H1, W1, K, H2), dev)
    _expect("grad_compressed_output_u", grad_compressed_output_u, (B, H1, W1, K, H2), dev)
    _expect("grad_compressed_output_v", grad_compressed_output_v, (B, H1, W1, K, W2), dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        d1 = torch.empty_like(f1)
        d2 = torch.empty_like(f2)
        da_u = torch.empty_like(attention_weights_u)
        da_v = torch.empty_like(attention_weights_v)
        ws, n = _workspace(lib, (B, H1, W1, H2, W2, C), dev)
        _lib.check(lib.sepcorr_compression_backward(
            f1.data_ptr(), f2.data_ptr(), attention_weights_u.data_ptr(), attention_weights_v.data_ptr(),
            grad_compressed_output_u.data_ptr(), grad_compressed_output_v.data_ptr(),
            d1.data_ptr(), d2.data_ptr(), da_u.data_ptr(), da_v.data_ptr(),
            B, H1, W1, H2, W2, C, K, ws.data_ptr(), n, _stream()))
    return [d1, d2, da_u, da_v]


# --- not part of the reference's native module: both backward passes of one pyramid level in one

def compression_weight_gradients(img1_features_l0, img2_features_lk, attention_weights_u, attention_weights_v,
                                 grad_compressed_output_u, grad_compressed_output_v):
    """-> [grad_attention_u (B,H1,W1,K,W2), grad_attention_v (B,H1,W1,K,H2)]: compression_backward without the
    feature gradients (one sweep over the volume instead of three)."""
    f1, f2 = img1_features_l0, img2_features_lk
    B, H1, W1, H2, W2, C = _dims(f1, f2)
    dev = f1.device
    _check("attention_weights_u", attention_weights_u, ndim=5)
    K = attention_weights_u.shape[3]
    _expect("attention_weights_u", attention_weights_u, (B, H1, W1, K, W2), dev)
    _expect("attention_weights_v", attention_weights_v, (B, H1, W1, K, H2), dev)
    _expect("grad_compressed_output_u", grad_compressed_output_u, (B, H1, W1, K, H2), dev)
    _expect("grad_compressed_output_v", grad_compressed_output_v, (B, H1, W1, K, W2), dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        da_u = torch.empty_like(attention_weights_u)
        da_v = torch.empty_like(attention_weights_v)
        ws, wptr, n = _fwd_workspace(lib, (B, H1, W1, H2, W2, C), K, dev)
        _lib.check(lib.sepcorr_compression_backward(
            f1.data_ptr(), f2.data_ptr(), attention_weights_u.data_ptr(), attention_weights_v.data_ptr(),
            grad_compressed_output_u.data_ptr(), grad_compressed_output_v.data_ptr(),
            None, None, da_u.data_ptr(), da_v.data_ptr(), B, H1, W1, H2, W2, C, K, wptr, n, _stream()))
    return [da_u, da_v]


# --- attention compression with the softmax inside the operator (core/corr.py:437-448 takes the softmax in torch)

def _logit_dims(f1, f2, logits_u, logits_v):
    B, H1, W1, H2, W2, C = _dims(f1, f2)
    _check("logits_u", logits_u, ndim=5)
    K = logits_u.shape[3]
    _expect("logits_u", logits_u, (B, H1, W1, K, W2), f1.device)
    _expect("logits_v", logits_v, (B, H1, W1, K, H2), f1.device)
    return B, H1, W1, H2, W2, C, K


def compression_forward_from_logits(img1_features_l0, img2_features_lk, logits_u, logits_v, stats_u=None, stats_v=None):
    """compression_forward with attention_weights = softmax(logits, dim=-1), the softmax taken inside the sweep.
    -> [compression_output_u, compression_output_v, stats_u (B,H1,W1,K,2), stats_v]: per row (max, sum of exp).
    Statistics a producer already has (attention_logits_forward) can be passed in; otherwise they are computed."""
    f1, f2 = img1_features_l0, img2_features_lk
    B, H1, W1, H2, W2, C, K = _logit_dims(f1, f2, logits_u, logits_v)
    dev = f1.device
    given = stats_u is not None and stats_v is not None
    lib = _lib.load()
    with torch.cuda.device(dev):
        cu = torch.empty((B, H1, W1, K, H2), dtype=f1.dtype, device=dev)
        cv = torch.empty((B, H1, W1, K, W2), dtype=f1.dtype, device=dev)
        if given:
            _expect("stats_u", stats_u, (B, H1, W1, K, 2), dev)
            _expect("stats_v", stats_v, (B, H1, W1, K, 2), dev)
        else:
            stats_u = torch.empty((B, H1, W1, K, 2), dtype=f1.dtype, device=dev)
            stats_v = torch.empty((B, H1, W1, K, 2), dtype=f1.dtype, device=dev)
        ws, wptr, n = _fwd_workspace(lib, (B, H1, W1, H2, W2, C), K, dev)
        _lib.check(lib.sepcorr_compression_forward_from_logits(
            f1.data_ptr(), f2.data_ptr(), logits_u.data_ptr(), logits_v.data_ptr(), cu.data_ptr(), cv.data_ptr(),
            stats_u.data_ptr(), stats_v.data_ptr(), int(given), B, H1, W1, H2, W2, C, K, wptr, n, _stream()))
    return [cu, cv, stats_u, stats_v]


def compression_backward_from_logits(img1_features_l0, img2_features_lk, logits_u, logits_v, stats_u, stats_v,
                                     compression_output_u, compression_output_v,
                                     grad_compressed_output_u, grad_compressed_output_v, need_features=True):
    """-> [grad_fmap1_l0, grad_fmap2_lk, grad_logits_u (B,H1,W1,K,W2), grad_logits_v (B,H1,W1,K,H2)]; the feature
    gradients are None with need_features=False (one sweep over the volume, no tensor of softmax outputs)."""
    f1, f2 = img1_features_l0, img2_features_lk
    B, H1, W1, H2, W2, C, K = _logit_dims(f1, f2, logits_u, logits_v)
    dev = f1.device
    _expect("stats_u", stats_u, (B, H1, W1, K, 2), dev)
    _expect("stats_v", stats_v, (B, H1, W1, K, 2), dev)
    _expect("compression_output_u", compression_output_u, (B, H1, W1, K, H2), dev)
    _expect("compression_output_v", compression_output_v, (B, H1, W1, K, W2), dev)
    _expect("grad_compressed_output_u", grad_compressed_output_u, (B, H1, W1, K, H2), dev)
    _expect("grad_compressed_output_v", grad_compressed_output_v, (B, H1, W1, K, W2), dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        d1 = torch.empty_like(f1) if need_features else None
        d2 = torch.empty_like(f2) if need_features else None
        dz_u = torch.empty_like(logits_u)
        dz_v = torch.empty_like(logits_v)
        n = lib.sepcorr_compression_backward_from_logits_workspace_bytes(B, H1, W1, H2, W2, C, K, int(need_features))
        ws = torch.empty(max(n, 1), dtype=torch.uint8, device=dev)
        _lib.check(lib.sepcorr_compression_backward_from_logits(
            f1.data_ptr(), f2.data_ptr(), logits_u.data_ptr(), logits_v.data_ptr(), stats_u.data_ptr(), stats_v.data_ptr(),
            compression_output_u.data_ptr(), compression_output_v.data_ptr(),
            grad_compressed_output_u.data_ptr(), grad_compressed_output_v.data_ptr(),
            d1.data_ptr() if need_features else None, d2.data_ptr() if need_features else None,
            dz_u.data_ptr(), dz_v.data_ptr(), B, H1, W1, H2, W2, C, K, ws.data_ptr(), n, _stream()))
    return [d1, d2, dz_u, dz_v]


def softmax_from_stats(logits, stats):
    """softmax(logits, dim=-1) from the saved row statistics (max, sum of exp): (.., L), (.., 2) -> (.., L)."""
    _check("logits", logits)
    L = logits.shape[-1]
    _expect("stats", stats, tuple(logits.shape[:-1]) + (2,), logits.device)
    lib = _lib.load()
    with torch.cuda.device(logits.device):
        a = torch.empty_like(logits)
        _lib.check(lib.sepcorr_softmax_rows(logits.data_ptr(), stats.data_ptr(), 1, a.data_ptr(),
                                            logits.numel() // L, L, _stream()))
    return a


def attention_logits_forward(sep, weight, bias, want_stats=True):
    """sep (B,H1,W1,2,L), Conv3d weight (K,2,3,3,3), bias (K) or None -> [logits (B,H1,W1,K,L), stats (B,H1,W1,K,2)]:
    the convolution alone, in the operator's layout, with the row statistics of its softmax."""
    _check("sep", sep, ndim=5)
    B, H1, W1, ch, L = sep.shape
    if ch != 2:
        raise RuntimeError(f"sep must have 2 channels (max, avg), got {ch}")
    _check("weight", weight, ndim=5)
    K = weight.shape[0]
    _expect("weight", weight, (K, 2, 3, 3, 3), sep.device)
    if bias is not None:
        _expect("bias", bias, (K,), sep.device)
    lib = _lib.load()
    with torch.cuda.device(sep.device):
        z = torch.empty((B, H1, W1, K, L), dtype=sep.dtype, device=sep.device)
        st = torch.empty((B, H1, W1, K, 2), dtype=sep.dtype, device=sep.device) if want_stats else None
        _lib.check(lib.sepcorr_attention_logits_forward(
            sep.data_ptr(), weight.data_ptr(), bias.data_ptr() if bias is not None else None, z.data_ptr(),
            st.data_ptr() if want_stats else None, B, H1, W1, L, K, _stream()))
    return [z, st]


def attention_logits_backward(sep, weight, grad_logits, need_bias=True):
    """-> [d_sep (B,H1,W1,2,L), d_weight (K,2,3,3,3), d_bias (K) or None] from the gradient of the logits."""
    _check("sep", sep, ndim=5)
    B, H1, W1, _, L = sep.shape
    K = weight.shape[0]
    _expect("weight", weight, (K, 2, 3, 3, 3), sep.device)
    _expect("grad_logits", grad_logits, (B, H1, W1, K, L), sep.device)
    lib = _lib.load()
    with torch.cuda.device(sep.device):
        d_sep = torch.empty_like(sep)
        d_w = torch.empty_like(weight)
        d_b = torch.empty(K, dtype=sep.dtype, device=sep.device) if need_bias else None
        n = lib.sepcorr_attention_logits_workspace_bytes(B, H1, W1, L, K)
        ws = torch.empty(max(n, 1), dtype=torch.uint8, device=sep.device)
        _lib.check(lib.sepcorr_attention_logits_backward(
            sep.data_ptr(), weight.data_ptr(), grad_logits.data_ptr(), d_sep.data_ptr(), d_w.data_ptr(),
            d_b.data_ptr() if need_bias else None, B, H1, W1, L, K, ws.data_ptr(), n, _stream()))
    return [d_sep, d_w, d_b]


def _att_levels_check(seps, weight, bias):
    for n, t in enumerate(seps):
        _check(f"seps[{n}]", t, ndim=5)
    B, H1, W1, ch, _ = seps[0].shape
    dev = seps[0].device
    for n, t in enumerate(seps):
        if tuple(t.shape[:4]) != (B, H1, W1, 2) or t.device != dev:
            raise RuntimeError(f"seps[{n}] must have shape ({B},{H1},{W1},2,L) on the same device")
    if not 1 <= len(seps) <= 4:
        raise RuntimeError("attention: 1 to 4 levels per call")
    _check("weight", weight, ndim=5)
    K = weight.shape[0]
    _expect("weight", weight, (K, 2, 3, 3, 3), dev)
    if bias is not None:
        _expect("bias", bias, (K,), dev)
    return B, H1, W1, K, dev


def attention_logits_forward_levels(seps, weight, bias):
    """attention_logits_forward for the max/avg volumes of several pyramid levels (same module: same weight and bias)
    in shared launches -> ([logits per level], [stats per level])."""
    import ctypes
    seps = list(seps)
    B, H1, W1, K, dev = _att_levels_check(seps, weight, bias)
    n = len(seps)
    lib = _lib.load()
    with torch.cuda.device(dev):
        zs = [torch.empty((B, H1, W1, K, t.shape[4]), dtype=t.dtype, device=dev) for t in seps]
        sts = [torch.empty((B, H1, W1, K, 2), dtype=t.dtype, device=dev) for t in seps]
        P = ctypes.c_void_p * n
        _lib.check(lib.sepcorr_attention_logits_forward_levels(
            P(*[t.data_ptr() for t in seps]), weight.data_ptr(), bias.data_ptr() if bias is not None else None,
            P(*[t.data_ptr() for t in zs]), P(*[t.data_ptr() for t in sts]), (ctypes.c_int * n)(*[t.shape[4] for t in seps]),
            n, B, H1, W1, K, _stream()))
    return zs, sts


def attention_logits_backward_levels(seps, weight, grad_logits, d_sep_init=None, need_bias=True):
    """attention_logits_backward for several levels of one module in shared launches -> ([d_sep per level], d_weight,
    d_bias or None), the weight and bias gradients summed over the levels; d_sep_init (optional, one tensor per level,
    shaped like seps) is added to the d_sep returned."""
    import ctypes
    seps, grad_logits = list(seps), list(grad_logits)
    B, H1, W1, K, dev = _att_levels_check(seps, weight, None)
    n = len(seps)
    for l in range(n):
        _expect(f"grad_logits[{l}]", grad_logits[l], (B, H1, W1, K, seps[l].shape[4]), dev)
        if d_sep_init is not None:
            _expect(f"d_sep_init[{l}]", d_sep_init[l], tuple(seps[l].shape), dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        d_seps = [torch.empty_like(t) for t in seps]
        d_w = torch.empty_like(weight)
        d_b = torch.empty(K, dtype=weight.dtype, device=dev) if need_bias else None
        Ls = (ctypes.c_int * n)(*[t.shape[4] for t in seps])
        nws = lib.sepcorr_attention_logits_levels_workspace_bytes(Ls, n, B, H1, W1, K)
        ws = torch.empty(max(nws, 1), dtype=torch.uint8, device=dev)
        P = ctypes.c_void_p * n
        _lib.check(lib.sepcorr_attention_logits_backward_levels(
            P(*[t.data_ptr() for t in seps]), weight.data_ptr(), P(*[t.data_ptr() for t in grad_logits]),
            P(*[t.data_ptr() for t in d_sep_init]) if d_sep_init is not None else None, P(*[t.data_ptr() for t in d_seps]),
            d_w.data_ptr(), d_b.data_ptr() if need_bias else None, Ls, n, B, H1, W1, K, ws.data_ptr(), nws, _stream()))
    return d_seps, d_w, d_b


# --- several pyramid levels per call (the caller's loop over levels, core/corr.py:416-457)

def _levels_setup(f1, f2_levels, K):
    import ctypes
    _check("img1_features_l0", f1, ndim=4)
    B, H1, W1, C = f1.shape
    lv = list(f2_levels)
    if not 1 <= len(lv) <= 4:
        raise RuntimeError("1 to 4 fmap2 levels are supported per call")
    for n, t in enumerate(lv):
        _check(f"img2_features_lvls[{n}]", t, ndim=4)
        if t.shape[0] != B or t.shape[3] != C or t.device != f1.device:
            raise RuntimeError(f"img2_features_lvls[{n}]: batch/feature size or device differs from img1_features_l0")
    L = len(lv)
    h2 = (ctypes.c_int * L)(*[t.shape[1] for t in lv])
    w2 = (ctypes.c_int * L)(*[t.shape[2] for t in lv])
    lib = _lib.load()
    n = lib.sepcorr_forward_levels_workspace_bytes(h2, w2, L, B, H1, W1, C, K)
    ws = torch.empty(max(n, 256), dtype=torch.uint8, device=f1.device)
    return lib, B, H1, W1, C, L, h2, w2, ws, n


def _ptrs(ts):
    import ctypes
    return (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])


def max_argmax_avg_forward_levels(img1_features_l0, img2_features_lvls):
    """max_argmax_avg_forward for every level of the fmap2 pyramid in one call -> list of [out_u, out_v, argmax_u, argmax_v]."""
    f1, lv = img1_features_l0, list(img2_features_lvls)
    lib, B, H1, W1, C, L, h2, w2, ws, n = _levels_setup(f1, lv, 2)
    dev = f1.device
    with torch.cuda.device(dev):
        ou = [torch.empty((B, H1, W1, 2, t.shape[1]), dtype=f1.dtype, device=dev) for t in lv]
        ov = [torch.empty((B, H1, W1, 2, t.shape[2]), dtype=f1.dtype, device=dev) for t in lv]
        au = [torch.empty((B, H1, W1, 1, t.shape[1]), dtype=torch.int32, device=dev) for t in lv]
        av = [torch.empty((B, H1, W1, 1, t.shape[2]), dtype=torch.int32, device=dev) for t in lv]
        _lib.check(lib.sepcorr_max_argmax_avg_forward_levels(f1.data_ptr(), _ptrs(lv), h2, w2, L, _ptrs(ou), _ptrs(ov), _ptrs(au),
                                                             _ptrs(av), B, H1, W1, C, ws.data_ptr(), n, _stream()))
    return [list(t) for t in zip(ou, ov, au, av)]


def _check_level_tensors(name, ts, lv, f1, K, which):
    B, H1, W1 = f1.shape[:3]
    for n, (t, f2) in enumerate(zip(ts, lv)):
        last = {"u": f2.shape[1], "v": f2.shape[2], "s": 2}[which]
        _expect(f"{name}[{n}]", t, (B, H1, W1, K, last), f1.device)


def compression_forward_from_logits_levels(img1_features_l0, img2_features_lvls, logits_u, logits_v, stats_u, stats_v):
    """compression_forward_from_logits (statistics given) for every level in one call -> list of [comp_u, comp_v]."""
    f1, lv = img1_features_l0, list(img2_features_lvls)
    K = logits_u[0].shape[3]
    lib, B, H1, W1, C, L, h2, w2, ws, n = _levels_setup(f1, lv, K)
    dev = f1.device
    _check_level_tensors("logits_u", logits_u, lv, f1, K, "v"); _check_level_tensors("logits_v", logits_v, lv, f1, K, "u")
    _check_level_tensors("stats_u", stats_u, lv, f1, K, "s"); _check_level_tensors("stats_v", stats_v, lv, f1, K, "s")
    with torch.cuda.device(dev):
        cu = [torch.empty((B, H1, W1, K, t.shape[1]), dtype=f1.dtype, device=dev) for t in lv]
        cv = [torch.empty((B, H1, W1, K, t.shape[2]), dtype=f1.dtype, device=dev) for t in lv]
        _lib.check(lib.sepcorr_compression_forward_from_logits_levels(
            f1.data_ptr(), _ptrs(lv), h2, w2, L, _ptrs(logits_u), _ptrs(logits_v), _ptrs(stats_u), _ptrs(stats_v),
            _ptrs(cu), _ptrs(cv), B, H1, W1, C, K, ws.data_ptr(), n, _stream()))
    return [list(t) for t in zip(cu, cv)]


def compression_logit_gradients_levels(img1_features_l0, img2_features_lvls, logits_u, logits_v, stats_u, stats_v,
                                       compression_output_u, compression_output_v, grad_compressed_output_u,
                                       grad_compressed_output_v):
    """The logit gradients of compression_backward_from_logits for every level in one call -> list of [dz_u, dz_v]."""
    f1, lv = img1_features_l0, list(img2_features_lvls)
    K = logits_u[0].shape[3]
    lib, B, H1, W1, C, L, h2, w2, ws, n = _levels_setup(f1, lv, K)
    _check_level_tensors("logits_u", logits_u, lv, f1, K, "v"); _check_level_tensors("logits_v", logits_v, lv, f1, K, "u")
    _check_level_tensors("stats_u", stats_u, lv, f1, K, "s"); _check_level_tensors("stats_v", stats_v, lv, f1, K, "s")
    _check_level_tensors("compression_output_u", compression_output_u, lv, f1, K, "u")
    _check_level_tensors("compression_output_v", compression_output_v, lv, f1, K, "v")
    _check_level_tensors("grad_compressed_output_u", grad_compressed_output_u, lv, f1, K, "u")
    _check_level_tensors("grad_compressed_output_v", grad_compressed_output_v, lv, f1, K, "v")
    with torch.cuda.device(f1.device):
        dz_u = [torch.empty_like(t) for t in logits_u]
        dz_v = [torch.empty_like(t) for t in logits_v]
        _lib.check(lib.sepcorr_compression_backward_from_logits_levels(
            f1.data_ptr(), _ptrs(lv), h2, w2, L, _ptrs(logits_u), _ptrs(logits_v), _ptrs(stats_u), _ptrs(stats_v),
            _ptrs(compression_output_u), _ptrs(compression_output_v), _ptrs(grad_compressed_output_u),
            _ptrs(grad_compressed_output_v), _ptrs(dz_u), _ptrs(dz_v), B, H1, W1, C, K, ws.data_ptr(), n, _stream()))
    return [list(t) for t in zip(dz_u, dz_v)]


def fused_backward(img1_features_l0, img2_features_lk, argmax_output_u, argmax_output_v, grad_MaxAvg_u, grad_MaxAvg_v,
                   attention_weights_u, attention_weights_v, grad_compressed_output_u, grad_compressed_output_v,
                   add_to_grad_fmap1=None):
    """-> [grad_fmap1_l0, grad_fmap2_lk]: the sum of what max_argmax_avg_backward and compression_backward return
    for the features, from one contraction per output (dL/dS of both operators is added before it is used).
    add_to_grad_fmap1: a gradient of fmap1 from other pyramid levels; this level's is added to it in place and the
    tensor returned as grad_fmap1_l0."""
    f1, f2 = img1_features_l0, img2_features_lk
    B, H1, W1, H2, W2, C = _dims(f1, f2)
    dev = f1.device
    _check("attention_weights_u", attention_weights_u, ndim=5)
    K = attention_weights_u.shape[3]
    _expect("argmax_output_u", argmax_output_u, (B, H1, W1, 1, H2), dev, torch.int32)
    _expect("argmax_output_v", argmax_output_v, (B, H1, W1, 1, W2), dev, torch.int32)
    _expect("grad_MaxAvg_u", grad_MaxAvg_u, (B, H1, W1, 2, H2), dev)
    _expect("grad_MaxAvg_v", grad_MaxAvg_v, (B, H1, W1, 2, W2), dev)
    _expect("attention_weights_u", attention_weights_u, (B, H1, W1, K, W2), dev)
    _expect("attention_weights_v", attention_weights_v, (B, H1, W1, K, H2), dev)
    _expect("grad_compressed_output_u", grad_compressed_output_u, (B, H1, W1, K, H2), dev)
    _expect("grad_compressed_output_v", grad_compressed_output_v, (B, H1, W1, K, W2), dev)
    lib = _lib.load()
    with torch.cuda.device(dev):
        if add_to_grad_fmap1 is not None:
            _expect("add_to_grad_fmap1", add_to_grad_fmap1, tuple(f1.shape), dev)
        d1 = torch.empty_like(f1) if add_to_grad_fmap1 is None else add_to_grad_fmap1
        d2 = torch.empty_like(f2)
        ws, n = _workspace(lib, (B, H1, W1, H2, W2, C), dev)
        _lib.check((lib.sepcorr_fused_backward if add_to_grad_fmap1 is None else lib.sepcorr_fused_backward_add)(
            f1.data_ptr(), f2.data_ptr(), argmax_output_u.data_ptr(), argmax_output_v.data_ptr(),
            grad_MaxAvg_u.data_ptr(), grad_MaxAvg_v.data_ptr(),
            attention_weights_u.data_ptr(), attention_weights_v.data_ptr(),
            grad_compressed_output_u.data_ptr(), grad_compressed_output_v.data_ptr(),
            d1.data_ptr(), d2.data_ptr(), B, H1, W1, H2, W2, C, K, ws.data_ptr(), n, _stream()))
    return [d1, d2]


# --- not part of the reference's native module: the attention-weight producer the caller runs between
# --- the two operators (core/corr.py:437-446), fused and in the operator's layout

def attention_forward(sep, weight, bias):
    """sep (B,H1,W1,2,L), Conv3d weight (K,2,3,3,3), bias (K) or None -> softmax_L(conv3d) as (B,H1,W1,K,L)."""
    _check("sep", sep, ndim=5)
    B, H1, W1, ch, L = sep.shape
    if ch != 2:
        raise RuntimeError(f"sep must have 2 channels (max, avg), got {ch}")
    _check("weight", weight, ndim=5)
    K = weight.shape[0]
    _expect("weight", weight, (K, 2, 3, 3, 3), sep.device)
    if bias is not None:
        _expect("bias", bias, (K,), sep.device)
    lib = _lib.load()
    with torch.cuda.device(sep.device):
        a = torch.empty((B, H1, W1, K, L), dtype=sep.dtype, device=sep.device)
        _lib.check(lib.sepcorr_attention_forward(sep.data_ptr(), weight.data_ptr(), bias.data_ptr() if bias is not None else None,
                                                 a.data_ptr(), B, H1, W1, L, K, _stream()))
    return a


def attention_backward(sep, weight, a, grad_a, need_bias=True):
    """-> [d_sep (B,H1,W1,2,L), d_weight (K,2,3,3,3), d_bias (K) or None]"""
    _check("sep", sep, ndim=5)
    B, H1, W1, _, L = sep.shape
    K = weight.shape[0]
    _expect("weight", weight, (K, 2, 3, 3, 3), sep.device)
    _expect("a", a, (B, H1, W1, K, L), sep.device)
    _expect("grad_a", grad_a, (B, H1, W1, K, L), sep.device)
    lib = _lib.load()
    with torch.cuda.device(sep.device):
        d_sep = torch.empty_like(sep)
        d_w = torch.empty_like(weight)
        d_b = torch.empty(K, dtype=sep.dtype, device=sep.device) if need_bias else None
        n = lib.sepcorr_attention_workspace_bytes(B, H1, W1, L, K)
        ws = torch.empty(max(n, 1), dtype=torch.uint8, device=sep.device)
        _lib.check(lib.sepcorr_attention_backward(sep.data_ptr(), weight.data_ptr(), a.data_ptr(), grad_a.data_ptr(),
                                                  d_sep.data_ptr(), d_w.data_ptr(), d_b.data_ptr() if need_bias else None,
                                                  B, H1, W1, L, K, ws.data_ptr(), n, _stream()))
    return [d_sep, d_w, d_b]


def feature_pyramid_forward(fmap, num_levels, divisor=1.0):
    """fmap (B,C,H,W) -> [level 0 .. level num_levels-1], level l in (B, H >> l, W >> l, C): the permuted map divided
    by `divisor`, and its 2x2 average poolings (core/corr.py:376-382, 419-422)."""
    import ctypes
    _check("fmap", fmap, ndim=4)
    B, C, H, W = fmap.shape
    lib = _lib.load()
    with torch.cuda.device(fmap.device):
        out = [torch.empty((B, H >> l, W >> l, C), dtype=fmap.dtype, device=fmap.device) for l in range(num_levels)]
        ptrs = (ctypes.c_void_p * num_levels)(*[t.data_ptr() for t in out])
        _lib.check(lib.sepcorr_feature_pyramid_forward(fmap.data_ptr(), ptrs, B, C, H, W, num_levels, float(divisor),
                                                       _stream()))
    return out


def feature_pyramid_backward(grad_levels, divisor=1.0):
    """Gradients of the levels (layouts as above) -> gradient of the (B,C,H,W) map."""
    import ctypes
    for n, g in enumerate(grad_levels):
        _check(f"grad_levels[{n}]", g, ndim=4)
    B, H, W, C = grad_levels[0].shape
    for l, g in enumerate(grad_levels):
        if tuple(g.shape) != (B, H >> l, W >> l, C) or g.device != grad_levels[0].device:
            raise RuntimeError(f"feature pyramid: level {l} must have shape {(B, H >> l, W >> l, C)} on the same device")
    n = len(grad_levels)
    lib = _lib.load()
    with torch.cuda.device(grad_levels[0].device):
        out = torch.empty((B, C, H, W), dtype=grad_levels[0].dtype, device=grad_levels[0].device)
        ptrs = (ctypes.c_void_p * n)(*[g.data_ptr() for g in grad_levels])
        _lib.check(lib.sepcorr_feature_pyramid_backward(ptrs, out.data_ptr(), B, C, H, W, n, float(divisor), _stream()))
    return out


def _src_tables(shapes, ptrs):
    import ctypes
    n = len(shapes)
    return ((ctypes.c_void_p * n)(*ptrs), (ctypes.c_int * n)(*[s[3] for s in shapes]),
            (ctypes.c_int * n)(*[s[4] for s in shapes]))


def assemble_forward(srcs, L0):
    """srcs: operator outputs (B,H1,W1,ch_n,L_n) in channel order -> (B, sum ch_n, L0, H1, W1), each one
    transposed and linearly interpolated along its last axis to length L0 (align_corners=True)."""
    for n, t in enumerate(srcs):
        _check(f"srcs[{n}]", t, ndim=5)
    B, H1, W1 = srcs[0].shape[:3]
    CT = sum(t.shape[3] for t in srcs)
    lib = _lib.load()
    with torch.cuda.device(srcs[0].device):
        dst = torch.empty((B, CT, L0, H1, W1), dtype=srcs[0].dtype, device=srcs[0].device)
        for t in srcs:
            if tuple(t.shape[:3]) != (B, H1, W1) or t.device != dst.device:
                raise RuntimeError("assemble: all sources must share batch, H1, W1 and device")
        if len(srcs) <= 8:     # one launch for the whole volume
            ptrs, ch, li = _src_tables([t.shape for t in srcs], [t.data_ptr() for t in srcs])
            _lib.check(lib.sepcorr_assemble_forward_multi(ptrs, ch, li, len(srcs), dst.data_ptr(), B, H1, W1, CT, L0,
                                                          _stream()))
            return dst
        c0 = 0
        for t in srcs:
            _lib.check(lib.sepcorr_assemble_forward(t.data_ptr(), dst.data_ptr(), B, H1, W1, t.shape[3], t.shape[4],
                                                    CT, c0, L0, _stream()))
            c0 += t.shape[3]
    return dst


def assemble_backward(grad_dst, shapes):
    """grad_dst (B,CT,L0,H1,W1) -> list of gradients with the given source shapes (B,H1,W1,ch_n,L_n)."""
    _check("grad_dst", grad_dst, ndim=5)
    B, CT, L0, H1, W1 = grad_dst.shape
    lib = _lib.load()
    with torch.cuda.device(grad_dst.device):
        out = [torch.empty(shp, dtype=grad_dst.dtype, device=grad_dst.device) for shp in shapes]
        if len(out) <= 8:
            ptrs, ch, li = _src_tables(shapes, [g.data_ptr() for g in out])
            _lib.check(lib.sepcorr_assemble_backward_multi(grad_dst.data_ptr(), ptrs, ch, li, len(out), B, H1, W1, CT, L0,
                                                           _stream()))
            return out
        c0 = 0
        for shp, g in zip(shapes, out):
            _lib.check(lib.sepcorr_assemble_backward(grad_dst.data_ptr(), g.data_ptr(), B, H1, W1, shp[3], shp[4],
                                                     CT, c0, L0, _stream()))
            c0 += shp[3]
    return out


def _lookup_args(f1, lvls, coords):
    import ctypes
    _check("img1_features_l0", f1, ndim=4)
    B, H1, W1, C = f1.shape
    _expect("coords", coords, (B, 2, H1, W1), f1.device)
    if not lvls:
        raise RuntimeError("at least one fmap2 level is needed")
    for n, t in enumerate(lvls):
        _check(f"img2_features_lvls[{n}]", t, ndim=4)
        if t.shape[0] != B or t.shape[3] != C or t.device != f1.device:
            raise RuntimeError(f"img2_features_lvls[{n}]: batch/feature size or device differs from img1_features_l0")
    L = len(lvls)
    ptrs = (ctypes.c_void_p * L)(*[t.data_ptr() for t in lvls])
    h2 = (ctypes.c_int * L)(*[t.shape[1] for t in lvls])
    w2 = (ctypes.c_int * L)(*[t.shape[2] for t in lvls])
    return B, H1, W1, C, L, ptrs, h2, w2


def lookup_forward(img1_features_l0, img2_features_lvls, coords, radius, scale):
    """Windowed bilinear lookup of the correlation pyramid, never holding the 4D volume.

    img1_features_l0 (B,H1,W1,C) unscaled, img2_features_lvls: list of pooled NHWC fmap2 levels (B,H2_l,W2_l,C),
    coords (B,2,H1,W1) with x in channel 0 -> (B, levels*(2*radius+1)^2, H1, W1), multiplied by `scale`.
    Stands where the reference calls alt_cuda_corr.forward once per level (core/corr.py:497-509); not a function
    of the reference's MemorySaver module.
    """
    f1, lvls = img1_features_l0, list(img2_features_lvls)
    B, H1, W1, C, L, ptrs, h2, w2 = _lookup_args(f1, lvls, coords)
    n = 2 * int(radius) + 1
    lib = _lib.load()
    with torch.cuda.device(f1.device):
        out = torch.empty((B, L * n * n, H1, W1), dtype=f1.dtype, device=f1.device)
        _lib.check(lib.sepcorr_lookup_forward(f1.data_ptr(), ptrs, h2, w2, coords.data_ptr(), out.data_ptr(),
                                              B, H1, W1, C, L, int(radius), float(scale), _stream()))
    return out


def lookup_backward(img1_features_l0, img2_features_lvls, coords, grad_out, radius, scale):
    """Gradients of lookup_forward: -> [d_f1 (B,H1,W1,C), [d_f2 level (B,H2_l,W2_l,C) ...]].  coords get none."""
    import ctypes
    f1, lvls = img1_features_l0, list(img2_features_lvls)
    B, H1, W1, C, L, ptrs, h2, w2 = _lookup_args(f1, lvls, coords)
    n = 2 * int(radius) + 1
    _expect("grad_out", grad_out, (B, L * n * n, H1, W1), f1.device)
    lib = _lib.load()
    with torch.cuda.device(f1.device):
        d_f1 = torch.empty_like(f1)
        d_f2 = [torch.empty_like(t) for t in lvls]
        dptrs = (ctypes.c_void_p * L)(*[t.data_ptr() for t in d_f2])
        nws = lib.sepcorr_lookup_backward_workspace_bytes(h2, w2, B, H1, W1, C, L, int(radius))
        ws = torch.empty(max(nws, 1), dtype=torch.uint8, device=f1.device)
        _lib.check(lib.sepcorr_lookup_backward(f1.data_ptr(), ptrs, h2, w2, coords.data_ptr(), grad_out.data_ptr(),
                                               d_f1.data_ptr(), dptrs, B, H1, W1, C, L, int(radius), float(scale),
                                               ws.data_ptr(), nws, _stream()))
    return [d_f1, d_f2]


def _lookup1d_dims(corr, coords):
    _check("corr", corr, ndim=5)
    B, dim, L, H1, W1 = corr.shape
    _expect("coords", coords, (B, 2, H1, W1), corr.device)
    return B, dim, L, H1, W1


def lookup1d_forward(corr, coords, coord_channel, clamp_unit, num_levels, radius):
    """Lookup in one separated volume corr (B,dim,L,H1,W1) at coords[:, coord_channel]:
    -> (B, num_levels*dim*(2*radius+1), H1, W1), what CorrBlock1D.__call__ computes per volume (core/corr.py:565-624)."""
    B, dim, L, H1, W1 = _lookup1d_dims(corr, coords)
    n = 2 * int(radius) + 1
    lib = _lib.load()
    with torch.cuda.device(corr.device):
        out = torch.empty((B, int(num_levels) * dim * n, H1, W1), dtype=corr.dtype, device=corr.device)
        _lib.check(lib.sepcorr_lookup1d_forward(corr.data_ptr(), coords.data_ptr(), out.data_ptr(), B, dim, L, H1, W1,
                                                int(coord_channel), int(bool(clamp_unit)), int(num_levels), int(radius),
                                                _stream()))
    return out


def lookup1d_backward(coords, grad_out, shape, coord_channel, clamp_unit, num_levels, radius):
    """Gradient of lookup1d_forward with respect to corr (of the given shape (B,dim,L,H1,W1))."""
    B, dim, L, H1, W1 = shape
    n = 2 * int(radius) + 1
    _expect("coords", coords, (B, 2, H1, W1), grad_out.device)
    _expect("grad_out", grad_out, (B, int(num_levels) * dim * n, H1, W1), coords.device)
    lib = _lib.load()
    with torch.cuda.device(grad_out.device):
        d_corr = torch.empty(shape, dtype=grad_out.dtype, device=grad_out.device)
        _lib.check(lib.sepcorr_lookup1d_backward(coords.data_ptr(), grad_out.data_ptr(), d_corr.data_ptr(), B, dim, L,
                                                 H1, W1, int(coord_channel), int(bool(clamp_unit)), int(num_levels),
                                                 int(radius), _stream()))
    return d_corr


CONTRACT_FP32, CONTRACT_BF16X3 = 0, 1
MAXAVG_AUTO, MAXAVG_DENSE, MAXAVG_GATHER = 0, 1, 2


def set_max_avg_backward(mode):
    """How max_argmax_avg_backward computes its gradients: MAXAVG_DENSE (recompute the correlation tile by tile),
    MAXAVG_GATHER (fetch the feature rows the maxima chose and multiply the averages' gradients by line means; needs
    C % 4 == 0 and C <= 256, dense elsewhere) or MAXAVG_AUTO (whichever is faster for the sizes of the call).
    Process-wide; returns the previous mode.  Not a function of the reference."""
    return _lib.load().sepcorr_set_max_avg_backward(int(mode))


def set_contraction(mode):
    """Arithmetic of the forward sweeps' contraction: CONTRACT_FP32 (fp32 MFMA) or CONTRACT_BF16X3 (three bf16
    planes per operand, fp32 accumulation; C == 256 only, fp32 elsewhere).  Process-wide; returns the previous mode.
    Not a function of the reference."""
    return _lib.load().sepcorr_set_contraction(int(mode))

