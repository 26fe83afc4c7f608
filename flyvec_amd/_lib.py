"""ctypes binding of libflyvec_hip.so (declared in include/flyvec_hip.h).

The reference binds five CUDA shared objects the same way (flyvec/train_flyvec.py:62-139).
There is no CPU fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes as C
from pathlib import Path

import numpy as np

import os

# FLYVEC_HIP_LIB points at another build of the same library (e.g. one compiled with extra flags).
LIB_PATH = Path(os.environ.get("FLYVEC_HIP_LIB") or Path(__file__).resolve().parent / "lib" / "libflyvec_hip.so")

FV_OK, FV_ERR_INVALID, FV_ERR_HIP, FV_ERR_STATE, FV_ERR_DATA = range(5)
FV_TRAIN_KERNELS = 6
TRAIN_KERNEL_NAMES = ("gather_winner", "group_xx", "sparse_owners", "absmax_ds", "update", "slot_update")


class FlyvecError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"libflyvec_hip error {code}: {message}")
        self.code = code


class TrainConfig(C.Structure):
    """fv_train_config"""
    _fields_ = [
        ("vocab", C.c_uint64),
        ("hid", C.c_uint32),
        ("window", C.c_uint32),
        ("batch", C.c_uint32),
        ("tie_rule", C.c_uint32),
        ("initial_learning_rate", C.c_float),
        ("delta", C.c_float),
        ("prec", C.c_float),
        ("lmid", C.c_float),
        ("lbase", C.c_float),
        ("prune_duplicates", C.c_uint32),
    ]


_vp, _u64, _u32, _i32, _f32 = C.c_void_p, C.c_uint64, C.c_uint32, C.c_int, C.c_float
_pp = C.POINTER(C.c_void_p)

# name -> argtypes; every function returns int status except fv_last_error
SIGNATURES = {
    "fv_device_count": [C.POINTER(C.c_int)],
    "fv_set_device": [_i32],
    "fv_device_info": [C.c_char_p, C.c_size_t, C.POINTER(C.c_int), C.POINTER(_u64)],
    "fv_device_memory": [C.POINTER(_u64), C.POINTER(_u64)],
    "fv_host_alloc_pinned": [C.c_size_t, _pp],
    "fv_host_free_pinned": [_vp],
    "fv_dev_alloc": [C.c_size_t, _pp],
    "fv_dev_free": [_vp],
    "fv_dev_upload": [_vp, _vp, C.c_size_t],
    "fv_dev_download": [_vp, _vp, C.c_size_t],
    "fv_calibration_copy": [C.c_size_t, _u32, C.POINTER(_f32)],
    "fv_count_windows": [_vp, _u64, _u64, C.POINTER(_u64)],
    "fv_build_window_starts": [_vp, _u64, _u64, _vp, _u64],
    "fv_inverse_frequency": [_vp, _u64, _u64, _vp],
    "fv_inverse_frequency_static": [_vp, _u64, _u64, _vp],
    "fv_histogram_stops_from": [_u64],
    "fv_mask_tokens": [_vp, _u64, _vp, _u64, _u64],
    "fv_prune_windows": [_vp, _u64, _u64],
    "fv_trainer_create": [C.POINTER(TrainConfig), _pp],
    "fv_trainer_destroy": [_vp],
    "fv_trainer_set_corpus": [_vp, _vp, _u64, _vp, _u64],
    "fv_trainer_set_corpus_starts": [_vp, _vp, _u64, _vp, _u64],
    "fv_trainer_num_windows": [_vp, C.POINTER(_u64)],
    "fv_trainer_get_window_starts": [_vp, _vp, _u64],
    "fv_trainer_get_inverse_frequency": [_vp, _vp],
    "fv_trainer_set_weights": [_vp, _vp],
    "fv_trainer_get_weights": [_vp, _vp],
    "fv_trainer_shuffle": [_vp, _u64],
    "fv_trainer_set_permutation": [_vp, _vp, _u64],
    "fv_trainer_get_permutation": [_vp, _vp, _u64],
    "fv_trainer_step": [_vp, _u64, _u32, _f32],
    "fv_trainer_step_delta": [_vp, _u64, _u32, _f32, _f32],
    "fv_trainer_epoch_delta": [_vp, _u64, _u64, _vp],
    "fv_trainer_get_second_winners": [_vp, _vp, _u32],
    "fv_trainer_run_epoch": [_vp, _u64, _u64],
    "fv_trainer_epoch_eps": [_vp, _u64, _u64, C.POINTER(_f32)],
    "fv_trainer_set_stale_tail": [_vp, _u32],
    "fv_trainer_sync": [_vp],
    "fv_trainer_get_giveups_recovered": [_vp, C.POINTER(_u64)],
    "fv_trainer_set_dense_launches": [_vp, _u32],
    "fv_trainer_get_dense_launches": [_vp, C.POINTER(_u32)],
    "fv_trainer_get_dense_path_counts": [_vp, C.POINTER(_u64), C.POINTER(_u64)],
    "fv_trainer_set_wait_limit": [_vp, _u32],
    "fv_trainer_set_grouping_launch": [_vp, _u32],
    "fv_trainer_set_slot_regions": [_vp, _u32],
    "fv_trainer_set_light_blocks": [_vp, _u32],
    "fv_trainer_set_sentinel_list": [_vp, _u32],
    "fv_trainer_get_grouping_launch": [_vp, C.POINTER(_u32)],
    "fv_trainer_get_winners": [_vp, _vp, _u32],
    "fv_trainer_get_step_stats": [_vp, _vp, C.POINTER(_f32)],
    "fv_trainer_row_norms": [_vp, _u32, _vp],
    "fv_trainer_time_steps": [_vp, _u64, _u32, _f32, C.POINTER(_f32), C.POINTER(_f32)],
    "fv_trainer_time_steps_graph": [_vp, _u64, _u32, _f32, _u32, C.POINTER(_f32)],
    "fv_trainer_time_kernel": [_vp, _u32, _u32, C.POINTER(_f32)],
    "fv_hasher_create": [_vp, _u32, _u64, _pp],
    "fv_hasher_destroy": [_vp],
    "fv_hasher_normalize": [_vp, _f32],
    "fv_hasher_row_sumsq": [_vp, _vp],
    "fv_hasher_row_sum_pow": [_vp, _u32, _vp],
    "fv_hasher_scale_rows": [_vp, _vp],
    "fv_hasher_get_weights": [_vp, _vp],
    "fv_hash_targets": [_vp, _vp, _u64, _u32, _vp],
    "fv_hash_windows": [_vp, _vp, _u64, _u32, _u32, _vp, _vp],
    "fv_hash_windows_dev": [_vp, _vp, _u64, _u32, _u32, _vp, _vp],
    "fv_hasher_sync": [_vp],
    "fv_hasher_time_windows": [_vp, _vp, _u64, _u32, _u32, _vp, _vp, _u32, C.POINTER(_f32)],
}

_lib = None


def load():
    """Load the library (once). Raises if it was never built -- there is no other backend."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise FileNotFoundError(
                f"{LIB_PATH} not found: build it with `flyvec_compile` (python -m flyvec_amd.build); "
                "this package has no CPU implementation")
        lib = C.CDLL(str(LIB_PATH))
        lib.fv_last_error.restype = C.c_char_p
        lib.fv_last_error.argtypes = []
        for name, args in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = C.c_int
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc):
    if rc != FV_OK:
        raise FlyvecError(rc, load().fv_last_error().decode("utf-8", "replace"))


def ptr(a):
    """Address of a numpy array's buffer (None passes NULL)."""
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def device_count():
    n = C.c_int(0)
    check(load().fv_device_count(C.byref(n)))
    return n.value


def device_info():
    name = C.create_string_buffer(256)
    cus = C.c_int(0)
    mem = C.c_uint64(0)
    check(load().fv_device_info(name, 256, C.byref(cus), C.byref(mem)))
    return {"name": name.value.decode(), "compute_units": cus.value, "hbm_bytes": mem.value}


def device_memory():
    """(free, total) bytes of the current device."""
    free, total = C.c_uint64(0), C.c_uint64(0)
    check(load().fv_device_memory(C.byref(free), C.byref(total)))
    return free.value, total.value


def calibration_copy(nbytes, reps=5):
    """Mean milliseconds of a plain copy kernel reading and writing nbytes each."""
    ms = C.c_float(0)
    check(load().fv_calibration_copy(int(nbytes), int(reps), C.byref(ms)))
    return ms.value


class _PinnedBlock:
    """Page-locked host memory from fv_host_alloc_pinned, returned with fv_host_free_pinned."""

    def __init__(self, nbytes):
        p = C.c_void_p()
        check(load().fv_host_alloc_pinned(max(int(nbytes), 1), C.byref(p)))
        self.ptr = p

    def __del__(self):
        try:
            if self.ptr is not None and self.ptr.value:
                load().fv_host_free_pinned(self.ptr)
        except Exception:
            pass
        self.ptr = None


def pinned_empty(shape, dtype):
    """A numpy array over page-locked host memory: the device copies such buffers by DMA without
    staging, which is what lets the host-buffer entry points (fv_hash_windows, fv_hash_targets) overlap their
    copies with the kernel. The memory is returned when the array and its views are gone."""
    dtype = np.dtype(dtype)
    n = int(np.prod(shape))
    block = _PinnedBlock(n * dtype.itemsize)
    raw = (C.c_ubyte * max(n * dtype.itemsize, 1)).from_address(block.ptr.value)
    raw._owner = block  # the ctypes view is the array's base and keeps the block alive
    return np.frombuffer(raw, dtype=dtype, count=n).reshape(shape)


class DeviceBuffer:
    """A block of HBM owned through fv_dev_alloc / fv_dev_free."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(load().fv_dev_alloc(self.nbytes, C.byref(p)))
        self.ptr = p

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        check(load().fv_dev_upload(buf.ptr, ptr(a), a.nbytes))
        return buf

    def to_numpy(self, dtype, shape):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        check(load().fv_dev_download(ptr(out), self.ptr, out.nbytes))
        return out

    def free(self):
        if self.ptr is not None and self.ptr.value:
            load().fv_dev_free(self.ptr)
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
