"""chainer_amd: the MI355X (gfx950) ``hip`` backend for ChainerX, driven from Python.

``chainer_amd`` exposes the ChainerX routine surface (``add``, ``dot``, ``conv``, ``linear``,
``fixed_batch_norm``, ``max_pool``, ``take``, ``log_softmax`` ...) over the C ABI of
``libhipcx.so``; every routine decomposes into kernel calls exactly as the reference routine does.
"""
from chainer_amd import _lib
from chainer_amd._lib import (OutOfMemoryError, ChainerxError, DimensionError, DtypeError, ChainerxNotImplementedError, ChainerxIndexError,
                              BackendError, DeviceError)
from chainer_amd._array import (ndarray, array, to_numpy, synchronize, device_available, memory_arena, pool_stats,
                                free_unused_blocks)
from chainer_amd.routines import *  # noqa: F401,F403
from chainer_amd import routines

_lib.load()  # fail at import time if the kernel library has not been built
