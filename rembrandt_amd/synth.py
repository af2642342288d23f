"""Seeded synthetic tensors (host side), from the library's own counter-based generator.

Element i of stream (seed, stream_id) depends only on (seed, stream_id, i), so the same arrays
can be regenerated anywhere without shipping data files.
"""
import ctypes as C

import numpy as np

from . import _lib


def _ptr(a):
    return C.c_void_p(a.ctypes.data)


def uniform(seed, stream_id, shape, lo=0.0, hi=1.0):
    a = np.empty(shape, np.float32)
    _lib.check(_lib.lib().rh_rng_fill_uniform(seed, stream_id, _ptr(a), a.size, lo, hi), "rh_rng_fill_uniform")
    return a


def normal(seed, stream_id, shape, mean=0.0, std=1.0):
    a = np.empty(shape, np.float32)
    _lib.check(_lib.lib().rh_rng_fill_normal(seed, stream_id, _ptr(a), a.size, mean, std), "rh_rng_fill_normal")
    return a


def integers(seed, stream_id, shape, modulus):
    a = np.empty(shape, np.int32)
    _lib.check(_lib.lib().rh_rng_fill_int(seed, stream_id, _ptr(a), a.size, modulus), "rh_rng_fill_int")
    return a
