// Seeded host-side input generation for the test harness (the role of MatmulTest*::Rerand and
// SetConstant, matmul_test.h:160-168, :328-351). The reference seeds std::rand from time(NULL) and
// is unreproducible by design; only its distribution is kept: uniform[min, max) rounded to the
// element type. Here every element is a pure function of (seed, stream, index), so any thread order
// and any sub-range reproduces the same arrays.
#include <cmath>
#include <cstdint>
#include <cstring>

#include "../../include/ckopt.h"
#include "ck_common.h"
#include "ck_numeric.h"

namespace {

inline uint64_t stream_base(uint64_t seed, uint64_t stream_id) { return seed + stream_id * 0xD1342543DE82EF95ull; }

inline float u24(uint64_t base, int64_t i) { return (float)(ck::splitmix64_at(base, (uint64_t)i) >> 40) * (1.0f / 16777216.0f); }

inline int store(int dtype, void* out, int64_t i, float v) {
    switch (dtype) {
        case ck::CK_DT_F16: static_cast<uint16_t*>(out)[i] = ck::float_to_half_bits(v); return 0;
        case ck::CK_DT_BF16: static_cast<uint16_t*>(out)[i] = ck::float_to_bf16_bits(v); return 0;
        case ck::CK_DT_F32: static_cast<float*>(out)[i] = v; return 0;
        case ck::CK_DT_I32: static_cast<int32_t*>(out)[i] = (int32_t)v; return 0;
        default: return -1;
    }
}

inline bool dtype_ok(int dtype) { return dtype >= ck::CK_DT_F16 && dtype <= ck::CK_DT_I32; }

}  // namespace

extern "C" {

int ckopt_fill_uniform(int dtype, void* out, int64_t n, uint64_t seed, uint64_t stream_id, float lo, float hi) {
    if (!dtype_ok(dtype) || n < 0) return ck::CK_ERR_BAD_PARAM;
    if (!out && n) return ck::CK_ERR_NULL;
    const uint64_t base = stream_base(seed, stream_id);
    const float span = hi - lo;
    for (int64_t i = 0; i < n; ++i) store(dtype, out, i, lo + u24(base, i) * span);
    return ck::CK_OK;
}

int ckopt_fill_normal(int dtype, void* out, int64_t n, uint64_t seed, uint64_t stream_id, float mean, float stddev) {
    if (!dtype_ok(dtype) || n < 0) return ck::CK_ERR_BAD_PARAM;
    if (!out && n) return ck::CK_ERR_NULL;
    // Box-Muller on two independent 24-bit uniforms drawn from two sub-streams of the same element index
    const uint64_t b1 = stream_base(seed, stream_id), b2 = stream_base(seed ^ 0xA5A5A5A5A5A5A5A5ull, stream_id);
    for (int64_t i = 0; i < n; ++i) {
        const double u1 = ((double)(ck::splitmix64_at(b1, (uint64_t)i) >> 40) + 1.0) * (1.0 / 16777216.0);  // (0, 1]
        const double u2 = (double)(ck::splitmix64_at(b2, (uint64_t)i) >> 40) * (1.0 / 16777216.0);
        const double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925 * u2);
        store(dtype, out, i, (float)(mean + stddev * z));
    }
    return ck::CK_OK;
}

int ckopt_fill_int(int dtype, void* out, int64_t n, uint64_t seed, uint64_t stream_id, int lo, int hi_inclusive) {
    if (!dtype_ok(dtype) || n < 0 || hi_inclusive < lo) return ck::CK_ERR_BAD_PARAM;
    if (!out && n) return ck::CK_ERR_NULL;
    const uint64_t base = stream_base(seed, stream_id);
    const uint64_t span = (uint64_t)((int64_t)hi_inclusive - lo + 1);
    for (int64_t i = 0; i < n; ++i) {
        const uint64_t r = (ck::splitmix64_at(base, (uint64_t)i) >> 11) % span;
        store(dtype, out, i, (float)(lo + (int64_t)r));
    }
    return ck::CK_OK;
}

int ckopt_fill_constant(int dtype, void* out, int64_t n, float value) {
    if (!dtype_ok(dtype) || n < 0) return ck::CK_ERR_BAD_PARAM;
    if (!out && n) return ck::CK_ERR_NULL;
    for (int64_t i = 0; i < n; ++i) store(dtype, out, i, value);
    return ck::CK_OK;
}

}  // extern "C"
