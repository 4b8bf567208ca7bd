// Host-side helpers shared by the translation units of libascq: error string, argument checks, launch check.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/ascq.h"

namespace ascq {

// Records a message for ascq_last_error() and returns `code` so that `return fail(...)` reads naturally.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

inline size_t dtype_size(int dt)
{
    switch (dt) {
        case ASCQ_F16:
        case ASCQ_BF16: return 2;
        case ASCQ_F32:
        case ASCQ_I32: return 4;
        case ASCQ_I8: return 1;
        case ASCQ_U64: return 8;
        default: return 0;
    }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int launch_status(const char* what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        return fail(ASCQ_EHIP, "%s: %s", what, hipGetErrorString(e));
    }
    return ASCQ_OK;
}

// Compute units of the current device, looked up once per device (the first 64 devices are cached; any thread may
// call this).  256 when the query fails.
inline uint32_t device_compute_units()
{
    static int cached[64];
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        return 256u;
    }
    n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            n = 256;
        }
        __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
    }
    return static_cast<uint32_t>(n);
}

// Plan recording (ascq_matmul_w8a8_plan): while a plan is being recorded on this thread, every launch site of the int8
// matmul describes the launch it would make and returns true, and the caller then skips the launch.  The first note of
// a call fills the main fields; later ones (the kernel that sums partial results) only add to `launches`;
// plan_note_extra records the second tile shape that the same launch runs for the last partial round.
bool plan_recording();
bool plan_note(int kernel, uint32_t tile_m, uint32_t tile_n, uint32_t tile_k, uint32_t workgroups, uint32_t k_splits,
               uint32_t lds_bytes, size_t workspace_bytes);
bool plan_note_extra(uint32_t narrow_tile_n, uint32_t narrow_workgroups);
void plan_begin(ascq_matmul_plan* plan);
void plan_end();

#define ASCQ_REQUIRE(cond, code, ...)          \
    do {                                       \
        if (!(cond)) {                         \
            return ::ascq::fail(code, __VA_ARGS__); \
        }                                      \
    } while (0)

}  // namespace ascq
