"""go-metal optimizer step on AMD MI355X (gfx950).

The product is the C-ABI shared library ``libgometal_hip.so`` built from ``csrc/`` and
``host/`` (see ``include/gometal_hip.h`` and ``include/gometal_optimizer.h``).  This module
is the thin ctypes view of that ABI that the tests, the smoke check and the benchmark use:
one Python function per exported C function, same names, same arguments, same return codes.
It contains no arithmetic and no fallback: if the library has not been built, importing the
bridge raises.
"""
import ctypes
import os

import numpy as np

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libgometal_hip.so")

u = ctypes.c_size_t          # uintptr_t
up = ctypes.POINTER(u)
i = ctypes.c_int
ip = ctypes.POINTER(i)
f = ctypes.c_float
fp = ctypes.POINTER(f)
vp = ctypes.c_void_p

# name -> (restype, argtypes): every symbol include/gometal_hip.h declares
ABI = {
    "create_metal_device": (u, []),
    "destroy_metal_device": (None, [u]),
    "create_command_queue": (u, [u]),
    "release_command_queue": (None, [u]),
    "allocate_metal_buffer": (u, [u, i, i]),
    "deallocate_metal_buffer": (None, [u]),
    "zero_metal_buffer": (i, [u, u, i]),
    "zero_metal_buffer_mpsgraph": (i, [u, u, i]),
    "copy_data_to_metal_buffer": (i, [u, vp, i]),
    "copy_float32_array_to_metal_buffer": (i, [u, vp, i]),
    "copy_int32_array_to_metal_buffer": (i, [u, vp, i]),
    "copy_metal_buffer_to_float32_array": (i, [u, vp, i]),
    "copy_metal_buffer_to_int32_array": (i, [u, vp, i]),
    "convert_tensor_type": (i, [u, u, ip, i, i, i, u]),
    "copy_buffer_to_buffer_sync": (i, [u, u, i, i, i]),
    "execute_sgd_step_mpsgraph": (i, [u, up, up, up, i, ip, f, f, f, i, i]),
    "execute_adam_step_mpsgraph": (i, [u, up, up, up, up, i, ip, f, f, f, f, f, i]),
    "execute_adam_step_mpsgraph_pooled": (i, [u, up, up, up, up, i, ip, f, f, f, f, f, i, u]),
    "execute_rmsprop_step_mpsgraph": (i, [u, up, up, up, up, up, i, ip, f, f, f, f, f, ctypes.c_bool, i]),
    "execute_adagrad_step_mpsgraph": (i, [u, up, up, up, i, ip, f, f, f]),
    "execute_adagrad_step_mpsgraph_pooled": (i, [u, up, up, up, i, ip, f, f, f, u]),
    "execute_adadelta_step_mpsgraph": (i, [u, up, up, up, up, i, ip, f, f, f]),
    "execute_adadelta_step_mpsgraph_pooled": (i, [u, up, up, up, up, i, ip, f, f, f, u]),
    "execute_nadam_step_mpsgraph": (i, [u, up, up, up, up, i, ip, f, f, f, f, f, i]),
    "gm_synchronize": (i, [u]),
    "gm_last_error": (ctypes.c_char_p, []),
    "gm_buffer_length": (ctypes.c_size_t, [u]),
    "gm_bias_corrections": (None, [f, f, i, fp, fp]),
    "gm_nadam_mu_next": (f, [f, i]),
    "gm_amp_state_create": (u, [u, f, f, f, i]),
    "gm_amp_state_destroy": (None, [u]),
    "gm_amp_state_get": (i, [u, fp, ip]),
    "gm_amp_state_set": (i, [u, f, i]),
    "execute_adam_amp_step": (i, [u, up, up, up, up, up, i, ip, f, f, f, f, f, i, u, ip, fp, ip]),
    "gm_timer_start": (i, [u]),
    "gm_timer_stop": (f, [u]),
    "gm_fill_normal_f32": (i, [u, u, ctypes.c_size_t, ctypes.c_uint64, f, f]),
    "gm_fill_normal_f16": (i, [u, u, ctypes.c_size_t, ctypes.c_uint64, f, f, f]),
    "gm_copy_probe": (i, [u, u, u, ctypes.c_size_t]),
    "gm_set_tuning": (i, [i, i, i]),
}

_LIB = None


def load_library(path=LIB_PATH):
    """Loads the built library and types every exported function.  Raises if it is missing."""
    global _LIB
    if _LIB is not None:
        return _LIB
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(there is no CPU fallback)")
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in ABI.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _LIB = lib
    return lib


def handle_array(handles):
    """A C uintptr_t[] from Python ints (None / 0 = nil handle).  None -> NULL array."""
    if handles is None:
        return None
    return (u * len(handles))(*[int(h or 0) for h in handles])


def int_array(values):
    return (i * len(values))(*[int(v) for v in values])


class Device:
    """Convenience owner of a device handle plus numpy <-> buffer helpers (test harness side)."""

    def __init__(self):
        self.lib = load_library()
        self.handle = self.lib.create_metal_device()
        if not self.handle:
            raise RuntimeError("create_metal_device() returned nil: no usable GPU (" +
                               self.lib.gm_last_error().decode() + ")")
        self._owned = []

    # ---- buffers ----
    def alloc(self, nbytes, zero=False):
        h = self.lib.allocate_metal_buffer(self.handle, int(nbytes), 1)
        if not h:
            raise MemoryError(f"allocate_metal_buffer({nbytes}) failed: " +
                              self.lib.gm_last_error().decode())
        self._owned.append(h)
        if zero:
            rc = self.lib.zero_metal_buffer(self.handle, h, int(nbytes))
            assert rc == 0, rc
        return h

    def free(self, h):
        self.lib.deallocate_metal_buffer(h)
        if h in self._owned:
            self._owned.remove(h)

    def upload(self, h, array):
        a = np.ascontiguousarray(array)
        rc = self.lib.copy_data_to_metal_buffer(h, a.ctypes.data_as(vp), a.nbytes)
        if rc != 0:
            raise RuntimeError(f"copy_data_to_metal_buffer rc={rc}: " + self.lib.gm_last_error().decode())

    def from_numpy(self, array):
        a = np.ascontiguousarray(array)
        h = self.alloc(max(a.nbytes, 1))
        if a.nbytes:
            self.upload(h, a)
        return h

    def to_numpy(self, h, count, dtype=np.float32):
        dtype = np.dtype(dtype)
        out = np.empty(count, dtype=dtype)
        if count == 0:
            return out
        nbytes = out.nbytes
        # the ABI reads back 4-byte elements: round up, then trim
        words = (nbytes + 3) // 4
        tmp = np.empty(words, dtype=np.uint32)
        rc = self.lib.copy_metal_buffer_to_int32_array(h, tmp.ctypes.data_as(vp), words)
        if rc != 0:
            raise RuntimeError(f"copy_metal_buffer_to_int32_array rc={rc}: " +
                               self.lib.gm_last_error().decode())
        return tmp.view(np.uint8)[:nbytes].view(dtype).copy()

    def synchronize(self):
        rc = self.lib.gm_synchronize(self.handle)
        if rc != 0:
            raise RuntimeError(f"gm_synchronize rc={rc}: " + self.lib.gm_last_error().decode())

    def close(self):
        for h in list(self._owned):
            self.lib.deallocate_metal_buffer(h)
        self._owned.clear()
        if self.handle:
            self.lib.destroy_metal_device(self.handle)
            self.handle = 0
