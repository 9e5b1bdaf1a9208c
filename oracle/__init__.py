"""CPU checker for the saved-activation compression path (test infrastructure).

A ctypes face over ``oracle/gact_oracle.c`` (the C restatement of the reference
arithmetic) plus the padding / reshaping glue of ``gact/gact/ops.py:11-69``.
Only tests, the smoke check and the bench's CPU-baseline leg may import this
package; the shipped library never does.

All arrays are numpy; ``float16`` arrays are handed to C as raw 16-bit words.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libgact_oracle.so")

NOISE_CONST, NOISE_INJECT, NOISE_REF, NOISE_FAST = 0, 1, 2, 3
GROUP = 256


def build(force=False):
    """Compile the C restatement (and the reference's calc_precision.cc when the checkout is there)."""
    src = os.path.join(_HERE, "gact_oracle.c")
    stale = not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src)
    if force or stale:
        subprocess.run(["make", "-C", _HERE, "-B", "-s", "all"], check=True)
    return _LIB_PATH


def build_ref(reference="/root/reference"):
    """Compile oracle/_ref from the reference checkout; returns False when it is absent."""
    if not os.path.isdir(reference):
        return False
    subprocess.run(["make", "-C", _HERE, "ref", "REFERENCE=" + reference], check=True)
    return True


def load_ref_calc_precision():
    """The reference's own calc_precision (compiled unmodified), or None when oracle/_ref is not built."""
    import glob
    import importlib.util

    hits = glob.glob(os.path.join(_HERE, "_ref", "gact_ref_calc_precision*.so"))
    if not hits:
        return None
    import torch  # noqa: F401  (the module links against libtorch)

    spec = importlib.util.spec_from_file_location("gact_ref_calc_precision", hits[0])
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i32, i64, u64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_uint64
        L.gact_oracle_minimax.argtypes = [vp, i32, i64, i64, vp, vp]
        L.gact_oracle_scale.argtypes = [vp, vp, i32, i32, i64, vp]
        L.gact_oracle_philox4x32_10.argtypes = [vp, vp, vp]
        L.gact_oracle_philox4x32.argtypes = [vp, vp, i32, vp]
        L.gact_oracle_curand_uniform.argtypes = [ctypes.c_uint32]
        L.gact_oracle_curand_uniform.restype = ctypes.c_float
        L.gact_oracle_noise.argtypes = [i32, u64, i32, i64, i64, i64, vp]
        L.gact_oracle_pack.argtypes = [vp, vp, vp, i32, i32, i64, i64, i64, i32, u64, vp, vp]
        L.gact_oracle_unpack.argtypes = [vp, i32, vp, vp, i32, i64, i64, i64, vp]
        L.gact_oracle_quantize.argtypes = [vp, i32, i64, i32, i32, u64, vp, vp, vp, vp, vp]
        L.gact_oracle_calc_precision.argtypes = [vp, vp, vp, i64, ctypes.c_double]
        L.gact_oracle_calc_precision.restype = i32
        L.gact_oracle_mask_pack.argtypes = [vp, i64, vp]
        L.gact_oracle_mask_unpack.argtypes = [vp, i64, vp]
        L.gact_oracle_num_threads.restype = i32
        L.gact_oracle_set_num_threads.argtypes = [i32]
        for name in ("gact_oracle_h2f", "gact_oracle_h2f_sw"):
            getattr(L, name).argtypes = [ctypes.c_uint16]
            getattr(L, name).restype = ctypes.c_float
        for name in ("gact_oracle_f2h", "gact_oracle_f2h_sw"):
            getattr(L, name).argtypes = [ctypes.c_float]
            getattr(L, name).restype = ctypes.c_uint16
        _lib = L
    return _lib


def num_threads():
    """OpenMP threads the C loops run on."""
    return int(lib().gact_oracle_num_threads())


def set_num_threads(n):
    lib().gact_oracle_set_num_threads(int(n))


def _dt(a):
    if a.dtype == np.float32:
        return 0
    if a.dtype == np.float16:
        return 1
    raise TypeError("oracle handles float32 and float16, got %s" % a.dtype)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _c(a, dtype=None):
    return np.ascontiguousarray(a, dtype=dtype)


def minimax(x):
    """Per-row (min, max) of a 2-D array.  minimax_cuda_kernel.cu:23-89."""
    x = _c(x)
    n, d = x.shape
    mn = np.empty(n, x.dtype)
    mx = np.empty(n, x.dtype)
    lib().gact_oracle_minimax(_p(x), _dt(x), n, d, _p(mn), _p(mx))
    return mn, mx


def scale(mn, mx, bits):
    """scale = T(2^b-1)/(max-min+2e-6).  quantization_cuda_kernel.cu:23-35."""
    mn, mx = _c(mn), _c(mx)
    out = np.empty_like(mn)
    lib().gact_oracle_scale(_p(mn), _p(mx), _dt(mn), bits, mn.size, _p(out))
    return out


def philox4x32(ctr, key, rounds):
    ctr = _c(ctr, np.uint32)
    key = _c(key, np.uint32)
    out = np.empty(4, np.uint32)
    lib().gact_oracle_philox4x32(_p(ctr), _p(key), int(rounds), _p(out))
    return out


def philox4x32_10(ctr, key):
    return philox4x32(ctr, key, 10)


FAST_ROUNDS = 7   # Philox rounds of the fast noise stream


def curand_uniform(x):
    return float(lib().gact_oracle_curand_uniform(int(x) & 0xFFFFFFFF))


def noise(noise_mode, seed, bits, N, G=1, D=GROUP):
    """The uniforms a noise mode feeds each element, shaped like the data [N,G,D]."""
    u = np.empty((N, G, D), np.float32)
    lib().gact_oracle_noise(noise_mode, seed & 0xFFFFFFFFFFFFFFFF, bits, N, G, D, _p(u))
    return u


def packed_len(bits, N, G=1, D=GROUP):
    """Bytes the pack kernel writes (the reference allocates one more).  quantization_cuda_kernel.cu:88-91."""
    wpt = 8 // bits
    n_round = N + (wpt - N % wpt) % wpt
    return bits * n_round * G * D // 8


def pack(data, mn, sc, bits, noise_mode=NOISE_CONST, seed=0, noise_tensor=None):
    """pack_single_precision_kernel on [N,G,D] data with per-(n,g) min / scale.  quantization_cuda_kernel.cu:38-71."""
    data = _c(data)
    N, G, D = data.shape
    mn, sc = _c(mn, data.dtype), _c(sc, data.dtype)
    assert mn.size == N * G and sc.size == N * G
    if noise_mode == NOISE_INJECT:
        noise_tensor = _c(noise_tensor, np.float32)
        assert noise_tensor.size == data.size
    out = np.zeros(packed_len(bits, N, G, D), np.uint8)
    lib().gact_oracle_pack(_p(data), _p(mn), _p(sc), _dt(data), bits, N, G, D, noise_mode,
                           seed & 0xFFFFFFFFFFFFFFFF, _p(noise_tensor), _p(out))
    return out


def unpack(packed, bits, sc, mn, N, G=1, D=GROUP):
    """unpack_single_precision_kernel.  quantization_cuda_kernel.cu:149-177."""
    packed = _c(packed).view(np.uint8)
    sc, mn = _c(sc), _c(mn)
    out = np.empty((N, G, D), sc.dtype)
    lib().gact_oracle_unpack(_p(packed), bits, _p(sc), _p(mn), _dt(sc), N, G, D, _p(out))
    return out


def pad_groups(x):
    """Flatten and zero-pad to whole groups of 256.  gact/gact/ops.py:12-19."""
    flat = _c(x).reshape(-1)
    N = (flat.size + GROUP - 1) // GROUP
    if N * GROUP != flat.size:
        flat = np.concatenate([flat, np.zeros(N * GROUP - flat.size, flat.dtype)])
    return flat.reshape(N, GROUP)


def op_quantize(x, bits, noise_mode=NOISE_CONST, seed=0, noise_tensor=None):
    """gact/gact/ops.py:11-32,57-59 -> (packed uint8, bits, scale [N,1,1], min [N,1,1], max [N])."""
    groups = pad_groups(x)
    N = groups.shape[0]
    if bits == 32:
        mn = groups.min(axis=1).reshape(N, 1)
        return groups, 32, (groups.max(axis=1).reshape(N, 1) - mn), mn, None
    mn, mx = minimax(groups)
    sc = scale(mn, mx, bits)
    pk = pack(groups.reshape(N, 1, GROUP), mn, sc, bits, noise_mode, seed, noise_tensor)
    return pk, bits, sc.reshape(N, 1, 1), mn.reshape(N, 1, 1), mx


def op_dequantize(q, shape):
    """gact/gact/ops.py:34-47,61-69."""
    pk, bits, sc, mn = q[:4]
    numel = int(np.prod(shape))
    if bits == 32:
        return np.ascontiguousarray(pk.reshape(-1)[:numel].reshape(shape))
    N = (numel + GROUP - 1) // GROUP
    out = unpack(pk, bits, sc.reshape(-1), mn.reshape(-1), N, 1, GROUP)
    return np.ascontiguousarray(out.reshape(-1)[:numel].reshape(shape))


def calc_precision(b, C, w, target):
    """Greedy bit allocation; mutates and returns ``b`` like calc_precision.cc:66-118."""
    assert b.dtype == np.int32 and C.dtype == np.float32 and w.dtype == np.int64
    rc = lib().gact_oracle_calc_precision(_p(b), _p(C), _p(w), b.size, float(target))
    if rc != 0:
        raise RuntimeError("budget unreachable: every tensor is already at 1 bit")
    return b


def mask_pack(data):
    data = _c(data, np.uint8).reshape(-1)
    out = np.empty((data.size + 31) // 32, np.int32)
    lib().gact_oracle_mask_pack(_p(data), data.size, _p(out))
    return out


def mask_unpack(mask, n):
    mask = _c(mask, np.int32)
    out = np.empty(n, np.uint8)
    lib().gact_oracle_mask_unpack(_p(mask), n, _p(out))
    return out
