"""ctypes binding of libglide_probes.so (include/glide_hip_probes.h): the measurement yardsticks behind bench.py's
--copy-calibration / --valu-calibration / --atomic-calibration flags.  Not part of the product library."""
import ctypes as C
import os

from glide_amd import capi

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(capi.__file__)), "libglide_probes.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libglide_probes.so is not built: run `make -C glide_amd/csrc`")
        _lib = C.CDLL(LIB_PATH)
    return _lib


def copy_bytes(dst, src, nbytes, stream=None):
    capi.check(lib().glide_probe_copy_bytes(capi._ptr(dst), capi._ptr(src), C.c_size_t(nbytes), C.c_void_p(stream)), "glide_probe_copy_bytes")


def valu_probe(mode, rounds, out, stream=None):
    capi.check(lib().glide_probe_valu(C.c_int(mode), C.c_uint32(rounds), capi._ptr(out), C.c_void_p(stream)), "glide_probe_valu")


def atomic_probe(mode, table, slots, rounds, out, stream=None):
    capi.check(lib().glide_probe_atomic(C.c_int(mode), capi._ptr(table), C.c_uint32(slots), C.c_uint32(rounds), capi._ptr(out), C.c_void_p(stream)),
               "glide_probe_atomic")


def gather_probe(table, row_count, row_bytes, row_stride_bytes, waves, rows_per_wave, rows_per_step, out, stream=None):
    capi.check(lib().glide_probe_gather(capi._ptr(table), C.c_uint32(row_count), C.c_uint32(row_bytes), C.c_uint32(row_stride_bytes), C.c_uint32(waves), C.c_uint32(rows_per_wave),
                                        C.c_int(rows_per_step), capi._ptr(out), C.c_void_p(stream)), "glide_probe_gather")
