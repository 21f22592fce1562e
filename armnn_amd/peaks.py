"""What this device delivers at its actual clocks: int8 MFMA issue rate and HBM copy rate (micro-benchmarks in
csrc/peaks.hip, built as lib/libmi355x_peaks.so).  Context for roofline fractions, which are quoted against the
published peaks."""
from __future__ import annotations

import ctypes as C
import os

_LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libmi355x_peaks.so")


def measure(copy_bytes: int = 1 << 30) -> dict:
    if not os.path.exists(_LIB):
        raise RuntimeError(f"{_LIB} is missing: build it with `make -C armnn_amd/csrc`")
    lib = C.CDLL(_LIB)
    lib.mi355x_peak_mfma_i8.argtypes = [C.c_int, C.POINTER(C.c_double)]
    lib.mi355x_peak_hbm_copy.argtypes = [C.c_size_t, C.POINTER(C.c_double)]
    lib.mi355x_peak_hbm_read.argtypes = [C.c_size_t, C.POINTER(C.c_double)]
    out = {}
    best = 0.0
    for waves in (1, 2, 4):
        v = C.c_double()
        rc = lib.mi355x_peak_mfma_i8(waves, C.byref(v))
        if rc != 0:
            raise RuntimeError(f"mi355x_peak_mfma_i8 failed ({rc})")
        best = max(best, v.value)
    out["mfma_i8_TOPs"] = best / 1e12
    # register-only chains again, with small and with full-range operand bytes, and the clock the device held meanwhile
    lib.mi355x_peak_mfma_i8_data.argtypes = [C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]
    for spread, key in ((0, "small_operands"), (1, "full_range_operands")):
        v, g = C.c_double(), C.c_double()
        rc = lib.mi355x_peak_mfma_i8_data(spread, C.byref(v), C.byref(g))
        if rc != 0:
            raise RuntimeError(f"mi355x_peak_mfma_i8_data failed ({rc})")
        out[f"mfma_i8_{key}_TOPs"] = v.value / 1e12
        out[f"mfma_i8_{key}_clock_GHz"] = g.value
    lib.mi355x_peak_mfma_i8_lds_fed.argtypes = [C.POINTER(C.c_double)]
    v = C.c_double()
    rc = lib.mi355x_peak_mfma_i8_lds_fed(C.byref(v))
    if rc != 0:
        raise RuntimeError(f"mi355x_peak_mfma_i8_lds_fed failed ({rc})")
    out["mfma_i8_lds_fed_TOPs"] = v.value / 1e12
    v = C.c_double()
    rc = lib.mi355x_peak_hbm_read(copy_bytes, C.byref(v))
    if rc != 0:
        raise RuntimeError(f"mi355x_peak_hbm_read failed ({rc})")
    out["hbm_read_GBps"] = v.value / 1e9
    v = C.c_double()
    rc = lib.mi355x_peak_hbm_copy(copy_bytes, C.byref(v))
    if rc != 0:
        raise RuntimeError(f"mi355x_peak_hbm_copy failed ({rc})")
    out["hbm_copy_GBps"] = v.value / 1e9
    return out


if __name__ == "__main__":
    import json
    print(json.dumps(measure()))
