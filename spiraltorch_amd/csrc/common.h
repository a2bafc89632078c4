// Shared host-side helpers for libsthip: thread-local error text, status plumbing and the
// checked-arithmetic validators every entry point uses.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "st_hip.h"

namespace sthip {

// Records `code`'s message for the calling thread and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// Formats a HIP failure the way the reference does: "{ctx}: {name} ({rc}) - {text}"
// (crates/st-backend-hip/src/real.rs:166-173).
int hip_fail(hipError_t rc, const char *ctx);
void clear_error();

// st_backend_hip::init(): returns ST_HIP_OK once a gfx950 device is usable.
int ensure_init();

inline bool checked_mul(size_t a, size_t b, size_t *out)
{
    if (b != 0 && a > static_cast<size_t>(-1) / b) return false;
    *out = a * b;
    return true;
}

constexpr size_t kMaxDim = 0x7fffffffu;  // dims must fit i32 (crates/st-tensor/src/backend/hip_dense.rs:55-73)

inline hipStream_t as_stream(void *stream) { return static_cast<hipStream_t>(stream); }

// Rows of A per launch when an A of 2 GiB or more is cut into row blocks for kernels that address their operands
// through 32-bit byte offsets: the largest multiple of 256 rows whose k·element_bytes bytes stay below 2^31, or 0 when
// not even 256 rows fit (the caller then leaves the product to a kernel with 64-bit addressing).
inline size_t gemm_row_block(size_t k, size_t element_bytes)
{
    const size_t row_bytes = k * element_bytes;
    if (row_bytes == 0) return 0;
    const size_t rows = ((1ull << 31) - 1) / row_bytes;  // rows·row_bytes <= 2^31 - 1
    return rows / 256 * 256;
}

}  // namespace sthip

#define ST_HIP_TRY(expr, ctx)                                        \
    do {                                                             \
        hipError_t st_rc_ = (expr);                                  \
        if (st_rc_ != hipSuccess) return ::sthip::hip_fail(st_rc_, ctx); \
    } while (0)

#define ST_HIP_CHECK(expr)                 \
    do {                                   \
        int st_status_ = (expr);           \
        if (st_status_ != ST_HIP_OK) return st_status_; \
    } while (0)
