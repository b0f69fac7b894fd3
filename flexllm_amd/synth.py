"""Seeded synthetic tensors: a counter-based PRNG (SplitMix64 of seed+index) that the host (numpy) and the
device fill kernels evaluate identically, so the CPU box and the GPU box see the same inputs."""
import ctypes as C

import numpy as np

from ._lib import lib, check
from .device import DeviceArray, _s

_M = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(seed, n, start=0):
    idx = np.arange(start + 1, start + n + 1, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + idx * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def _u01(z):
    return (z >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / 16777216.0)


def host_i8(shape, seed, lo=-127, hi=127):
    n = int(np.prod(shape))
    z = splitmix64(seed, n)
    return (lo + ((z >> np.uint64(33)) % np.uint64(hi - lo + 1)).astype(np.int64)).astype(np.int8).reshape(shape)


def host_uniform_f32(shape, seed, lo, hi):
    n = int(np.prod(shape))
    u = _u01(splitmix64(seed, n))
    return (np.float32(lo) + (np.float32(hi) - np.float32(lo)) * u).astype(np.float32).reshape(shape)


def host_uniform_f16(shape, seed, lo, hi):
    return host_uniform_f32(shape, seed, lo, hi).astype(np.float16)


def host_normal_f32(shape, seed):
    """Box-Muller on two SplitMix64 streams (host only; activations are uploaded)."""
    n = int(np.prod(shape))
    u1 = _u01(splitmix64(seed, n)).astype(np.float64)
    u2 = _u01(splitmix64(seed ^ 0x5DEECE66D, n)).astype(np.float64)
    r = np.sqrt(-2.0 * np.log(1.0 - u1))
    return (r * np.cos(2.0 * np.pi * u2)).astype(np.float32).reshape(shape)


def device_i8(shape, seed, lo=-127, hi=127, stream=None):
    a = DeviceArray(shape, np.int8)
    check(lib().flexllm_rt_fill_i8(C.c_void_p(a.ptr), C.c_size_t(a.size), C.c_uint64(seed), lo, hi, _s(stream)))
    return a


def device_uniform_f32(shape, seed, lo, hi, stream=None):
    a = DeviceArray(shape, np.float32)
    check(lib().flexllm_rt_fill_uniform_f32(C.c_void_p(a.ptr), C.c_size_t(a.size), C.c_uint64(seed),
                                            C.c_float(lo), C.c_float(hi), _s(stream)))
    return a


def device_uniform_f16(shape, seed, lo, hi, stream=None):
    a = DeviceArray(shape, np.float16)
    check(lib().flexllm_rt_fill_uniform_f16(C.c_void_p(a.ptr), C.c_size_t(a.size), C.c_uint64(seed),
                                            C.c_float(lo), C.c_float(hi), _s(stream)))
    return a
