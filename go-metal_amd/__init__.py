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
    "execute_lbfgs_step_mpsgraph": (i, [u, up, up, up, up, up, up, up, u, i, ip, i, i, i, f, f, f, i, f, f, fp]),
    "execute_lbfgs_step_mpsgraph_pooled": (i, [u, up, up, up, up, up, up, up, u, i, ip, i, i, i, f, f, f, i, f, f,
                                               u, fp]),
    "gm_lbfgs_dot": (i, [u, up, up, i, ip, fp]),
    "gm_synchronize": (i, [u]),
    "gm_wait_for_stream": (i, [u, vp]),
    "gm_signal_stream": (i, [u, vp]),
    "gm_last_error": (ctypes.c_char_p, []),
    "gm_buffer_length": (ctypes.c_size_t, [u]),
    "gm_bias_corrections": (None, [f, f, i, fp, fp]),
    "gm_nadam_mu_next": (f, [f, i]),
    "gm_amp_state_create": (u, [u, f, f, f, i]),
    "gm_amp_state_destroy": (None, [u]),
    "gm_amp_state_get": (i, [u, fp, ip]),
    "gm_amp_state_set": (i, [u, f, i]),
    "gm_amp_state_query": (i, [u, fp, ip, ip, ip]),
    "gm_amp_state_set_step_count": (i, [u, i]),
    "gm_amp_state_max_in_flight": (i, [u]),
    "execute_adam_amp_step_async": (i, [u, up, up, up, up, up, i, ip, f, f, f, f, f, u]),
    "execute_adam_amp_step": (i, [u, up, up, up, up, up, i, ip, f, f, f, f, f, i, u, ip, fp, ip]),
    "gm_allocate_buffer_phased": (u, [u, i, i, i]),
    "execute_adam_step_noalloc": (i, [u, up, up, up, up, i, ip, f, f, f, f, f, i]),
    "gm_plan_cache_stats": (i, [u, ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64), ip]),
    "execute_adam_amp_step_fused": (i, [u, up, up, up, up, up, up, up, up, i, ip, f, f, f, f, f, i, u, ip, fp, ip, ip]),
    "execute_adam_amp_step_fused_async": (i, [u, up, up, up, up, up, up, up, up, i, ip, f, f, f, f, f, u]),
    "gm_amp_state_current_set": (i, [u]),
    "gm_amp_state_set_current_set": (i, [u, i]),
    "gm_timer_start": (i, [u]),
    "gm_timer_stop": (f, [u]),
    "gm_fill_normal_f32": (i, [u, u, ctypes.c_size_t, ctypes.c_uint64, f, f]),
    "gm_fill_normal_f16": (i, [u, u, ctypes.c_size_t, ctypes.c_uint64, f, f, f]),
    "gm_copy_probe": (i, [u, u, u, ctypes.c_size_t]),
    "gm_set_tuning": (i, [u, i, i, i]),
    "gm_set_workgroup_lanes": (i, [u, i]),
    "gm_set_amp_check_order": (i, [u, i, i]),
}

# name -> (restype, argtypes): every symbol include/gometal_optimizer.h declares
c_str = ctypes.c_char_p
HOST_ABI = {
    "gmo_last_error": (c_str, []),
    "gmo_free_string": (None, [vp]),
    "gmo_memory_manager_new": (u, [u]),
    "gmo_memory_manager_free": (None, [u]),
    "gmo_initialize_global_memory_manager": (None, [u]),
    "gmo_get_global_memory_manager": (u, []),
    "gmo_allocate_buffer": (u, [u, i]),
    "gmo_release_buffer": (None, [u, u]),
    "gmo_find_pool_size": (i, [u, i]),
    "gmo_calculate_max_pool_size": (i, [i]),
    "gmo_reference_max_pool_size": (i, [i]),
    "gmo_set_pool_byte_budget": (None, [ctypes.c_size_t]),
    "gmo_pool_stats": (i, [u, i, ip, ip, ip]),
    "gmo_default_config": (i, [fp]),
    "gmo_optimizer_new": (u, [i, fp, ip, ip, i, u, u]),
    "gmo_optimizer_free": (None, [u]),
    "gmo_set_weight_buffers": (i, [u, up, i]),
    "gmo_step": (i, [u, up, i]),
    "gmo_get_step_count": (ctypes.c_uint64, [u]),
    "gmo_update_learning_rate": (None, [u, f]),
    "gmo_set_command_pool": (None, [u, u]),
    "gmo_cleanup": (None, [u]),
    "gmo_get_state_json": (vp, [u]),
    "gmo_load_state_json": (i, [u, c_str]),
    "gmo_state_json_normalize": (vp, [c_str]),
    "gmo_extract_float32_param": (f, [c_str, c_str, f]),
    "gmo_extract_bool_param": (i, [c_str, c_str, i]),
    "gmo_extract_uint64_param": (ctypes.c_uint64, [c_str, c_str, ctypes.c_uint64]),
    "gmo_validate_state_type": (i, [c_str, c_str]),
    "gmo_restore_buffer_state": (i, [u, fp, i, i, c_str]),
    "gmo_extract_buffer_state": (i, [u, i, c_str, c_str, fp, i]),
    "gmo_get_checkpoint_json": (vp, [u]),
    "gmo_load_checkpoint_json": (i, [u, c_str]),
    "gmo_get_field": (f, [u, c_str]),
    "gmo_state_buffer": (u, [u, c_str, i]),
    "gmo_uses_pooling": (i, [u]),
    "gmo_set_log_progress": (None, [u, i]),
    "gmo_enable_mixed_precision": (i, [u, f, f, f, i]),
    "gmo_enable_ping_pong": (i, [u]),
    "gmo_current_set": (i, [u]),
    "gmo_step_amp": (i, [u, up, up, i, ip]),
    "gmo_step_amp_async": (i, [u, up, up, i]),
    "gmo_sync_amp": (i, [u, ctypes.POINTER(ctypes.c_uint64)]),
    "gmo_loss_scale": (f, [u]),
    "gmo_growth_tracker": (i, [u]),
    "gmo_lbfgs_default_config": (None, [ip, fp, ip, fp, fp, fp]),
    "gmo_lbfgs_new": (u, [i, f, i, f, f, f, ip, ip, i, u, u]),
    "gmo_lbfgs_free": (None, [u]),
    "gmo_lbfgs_set_weight_buffers": (i, [u, up, i]),
    "gmo_lbfgs_step": (i, [u, up, i, f]),
    "gmo_lbfgs_set_command_pool": (None, [u, u]),
    "gmo_lbfgs_uses_pooling": (i, [u]),
    "gmo_lbfgs_get_step": (ctypes.c_uint64, [u]),
    "gmo_lbfgs_get_stats": (None, [u, ctypes.POINTER(ctypes.c_uint64), ip, ip, fp]),
    "gmo_lbfgs_history": (None, [u, ip, ip, fp]),
    "gmo_lbfgs_cleanup": (None, [u]),
    "gmo_lbfgs_update_learning_rate": (i, [u, f]),
    "gmo_lbfgs_set_log_progress": (None, [u, i]),
    "gmo_lbfgs_buffer_size": (i, [u, i]),
    "gmo_lbfgs_buffer": (u, [u, c_str, i, i]),
    "gmo_tensor_new": (u, [ip, i, i, i]),
    "gmo_tensor_retain": (u, [u]),
    "gmo_tensor_release": (None, [u]),
    "gmo_tensor_free": (None, [u]),
    "gmo_tensor_buffer": (u, [u]),
    "gmo_tensor_size": (i, [u]),
    "gmo_tensor_ref_count": (i, [u]),
    "gmo_tensor_dtype": (i, [u]),
    "gmo_tensor_convert_to": (u, [u, i]),
    "gmo_tensor_copy_float32_data": (i, [u, vp, i]),
    "gmo_tensor_to_float32_slice": (i, [u, vp, i]),
    "gmo_tensor_string": (vp, [u]),
    "gmo_tensor_copy_from": (i, [u, u]),
    "gmo_calculate_size": (i, [ip, i, i]),
    "gmo_execute_step_with_precomputed_gradients": (i, [u, up, i, up, i]),
    "gmo_scheduler_new": (u, [i, i, ctypes.c_double, ctypes.c_double, c_str]),
    "gmo_scheduler_free": (None, [u]),
    "gmo_scheduler_get_lr": (ctypes.c_double, [u, i, i, ctypes.c_double]),
    "gmo_scheduler_plateau_step": (ctypes.c_double, [u, ctypes.c_double, ctypes.c_double]),
    "gmo_scheduler_name": (c_str, [u]),
    "gmo_scheduler_apply": (ctypes.c_double, [u, u, i, i, ctypes.c_double]),
    "gmo_pow": (f, [f, f]),
    "gmo_extract_buffer_index": (i, [c_str]),
    "gmo_calculate_tensor_size": (i, [ip, i]),
}
HOST_ABI["gmo_default_config"] = (i, [i, fp])
HOST_ABI_NAMES = set(HOST_ABI)

KINDS = {"sgd": 0, "adam": 1, "rmsprop": 2, "adagrad": 3, "adadelta": 4, "nadam": 5}

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
    for name, (restype, argtypes) in list(ABI.items()) + list(HOST_ABI.items()):
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
    def alloc(self, nbytes, zero=False, phase=None):
        """phase: start the buffer at this many bytes modulo 2 MiB (gm_allocate_buffer_phased)."""
        if phase is None:
            h = self.lib.allocate_metal_buffer(self.handle, int(nbytes), 1)
        else:
            h = self.lib.gm_allocate_buffer_phased(self.handle, int(nbytes), 1, int(phase))
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


class HostLBFGS:
    """Python handle on the C++ LBFGSOptimizerState (mirror of optimizer/lbfgs.go)."""

    def __init__(self, config, weight_shapes, memory_manager, device):
        """config: (HistorySize, LineSearchTol, MaxLineSearch, C1, C2, InitialStep)."""
        self.lib = load_library()
        dims = [int(d) for shape in weight_shapes for d in shape]
        ndims = [len(shape) for shape in weight_shapes]
        hs, tol, mls, c1, c2, step = config
        self.handle = self.lib.gmo_lbfgs_new(
            int(hs), tol, int(mls), c1, c2, step, int_array(dims) if dims else None,
            int_array(ndims) if ndims else None, len(weight_shapes), int(memory_manager or 0), int(device or 0))
        self.error = None if self.handle else self.lib.gmo_last_error().decode()
        if self.handle:
            self.lib.gmo_lbfgs_set_log_progress(self.handle, 0)

    @staticmethod
    def default_config():
        lib = load_library()
        hs, mls = ctypes.c_int(), ctypes.c_int()
        tol, c1, c2, step = f(), f(), f(), f()
        lib.gmo_lbfgs_default_config(ctypes.byref(hs), ctypes.byref(tol), ctypes.byref(mls), ctypes.byref(c1),
                                     ctypes.byref(c2), ctypes.byref(step))
        return hs.value, tol.value, mls.value, c1.value, c2.value, step.value

    def _err(self, rc):
        return None if rc == 0 else self.lib.gmo_last_error().decode()

    def SetWeightBuffers(self, buffers):
        return self._err(self.lib.gmo_lbfgs_set_weight_buffers(self.handle, handle_array(buffers), len(buffers)))

    def Step(self, gradient_buffers, current_loss):
        return self._err(self.lib.gmo_lbfgs_step(self.handle, handle_array(gradient_buffers),
                                                 len(gradient_buffers), current_loss))

    def SetCommandPool(self, pool):
        self.lib.gmo_lbfgs_set_command_pool(self.handle, int(pool or 0))

    def uses_pooling(self):
        return bool(self.lib.gmo_lbfgs_uses_pooling(self.handle))

    def GetStep(self):
        return self.lib.gmo_lbfgs_get_step(self.handle)

    def GetStats(self):
        step, hs, used, loss = ctypes.c_uint64(), ctypes.c_int(), ctypes.c_int(), f()
        self.lib.gmo_lbfgs_get_stats(self.handle, ctypes.byref(step), ctypes.byref(hs), ctypes.byref(used),
                                     ctypes.byref(loss))
        return {"step": step.value, "history_size": hs.value, "history_used": used.value,
                "prev_loss": loss.value}

    def history(self):
        count, index, step = ctypes.c_int(), ctypes.c_int(), f()
        self.lib.gmo_lbfgs_history(self.handle, ctypes.byref(count), ctypes.byref(index), ctypes.byref(step))
        return count.value, index.value, step.value

    def UpdateLearningRate(self, lr):
        return self._err(self.lib.gmo_lbfgs_update_learning_rate(self.handle, lr))

    def Cleanup(self):
        self.lib.gmo_lbfgs_cleanup(self.handle)

    def buffer(self, which, history=0, index=0):
        return self.lib.gmo_lbfgs_buffer(self.handle, which.encode(), history, index)

    def buffer_size(self, index):
        return self.lib.gmo_lbfgs_buffer_size(self.handle, index)

    def free(self):
        if self.handle:
            self.lib.gmo_lbfgs_free(self.handle)
            self.handle = 0


class HostOptimizer:
    """Python handle on one of the C++ optimizer objects (the mirror of the Go `optimizer`
    package), through include/gometal_optimizer.h.  Method names follow the Go methods."""

    def __init__(self, kind, config, weight_shapes, memory_manager, device):
        self.lib = load_library()
        self.kind = kind
        cfg = (f * 6)(*([float(x) for x in config] + [0.0] * (6 - len(config))))
        dims = [int(d) for shape in weight_shapes for d in shape]
        ndims = [len(shape) for shape in weight_shapes]
        self.handle = self.lib.gmo_optimizer_new(
            KINDS[kind], cfg, int_array(dims) if dims else None, int_array(ndims) if ndims else None,
            len(weight_shapes), int(memory_manager or 0), int(device or 0))
        self.error = None if self.handle else self.lib.gmo_last_error().decode()

    def _err(self, rc):
        return None if rc == 0 else self.lib.gmo_last_error().decode()

    def SetWeightBuffers(self, buffers):
        return self._err(self.lib.gmo_set_weight_buffers(self.handle, handle_array(buffers), len(buffers)))

    def Step(self, gradient_buffers):
        return self._err(self.lib.gmo_step(self.handle, handle_array(gradient_buffers), len(gradient_buffers)))

    def StepAMP(self, gradient16_buffers, weight16_buffers=None):
        skipped = ctypes.c_int(-1)
        rc = self.lib.gmo_step_amp(self.handle, handle_array(gradient16_buffers), handle_array(weight16_buffers),
                                   len(gradient16_buffers), ctypes.byref(skipped))
        return bool(skipped.value), self._err(rc)

    def StepAMPAsync(self, gradient16_buffers, weight16_buffers=None):
        return self._err(self.lib.gmo_step_amp_async(self.handle, handle_array(gradient16_buffers),
                                                     handle_array(weight16_buffers), len(gradient16_buffers)))

    def SyncAMP(self):
        skipped = ctypes.c_uint64(0)
        rc = self.lib.gmo_sync_amp(self.handle, ctypes.byref(skipped))
        return skipped.value, self._err(rc)

    def EnableMixedPrecision(self, initial_scale=65536.0, growth_factor=2.0, backoff_factor=0.5, growth_interval=2000):
        return self._err(self.lib.gmo_enable_mixed_precision(self.handle, initial_scale, growth_factor,
                                                             backoff_factor, growth_interval))

    def EnablePingPong(self):
        return self._err(self.lib.gmo_enable_ping_pong(self.handle))

    def current_set(self):
        return self.lib.gmo_current_set(self.handle)

    def GetStepCount(self):
        return self.lib.gmo_get_step_count(self.handle)

    def UpdateLearningRate(self, lr):
        self.lib.gmo_update_learning_rate(self.handle, lr)

    def SetCommandPool(self, pool):
        self.lib.gmo_set_command_pool(self.handle, int(pool or 0))

    def Cleanup(self):
        self.lib.gmo_cleanup(self.handle)

    def GetStateJSON(self):
        p = self.lib.gmo_get_state_json(self.handle)
        if not p:
            return None, self.lib.gmo_last_error().decode()
        text = ctypes.string_at(p).decode()
        self.lib.gmo_free_string(p)
        return text, None

    def LoadStateJSON(self, text):
        return self._err(self.lib.gmo_load_state_json(self.handle, text.encode()))

    def GetCheckpointJSON(self):
        p = self.lib.gmo_get_checkpoint_json(self.handle)
        if not p:
            return None, self.lib.gmo_last_error().decode()
        text = ctypes.string_at(p).decode()
        self.lib.gmo_free_string(p)
        return text, None

    def LoadCheckpointJSON(self, text):
        return self._err(self.lib.gmo_load_checkpoint_json(self.handle, text.encode()))

    def field(self, name):
        return self.lib.gmo_get_field(self.handle, name.encode())

    def state_buffer(self, state_type, index):
        return self.lib.gmo_state_buffer(self.handle, state_type.encode(), index)

    def free(self):
        if self.handle:
            self.lib.gmo_optimizer_free(self.handle)
            self.handle = 0
