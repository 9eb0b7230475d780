// Shared device/host helpers for libsnnf (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "snnf.h"

namespace snnf {

// ---------------------------------------------------------------------------------------------------------------
// Error reporting
// ---------------------------------------------------------------------------------------------------------------
char* last_error_buffer();  // thread-local, 512 bytes (defined in snnf_capi.hip)

inline int fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(last_error_buffer(), 512, fmt, ap);
    va_end(ap);
    return status;
}

inline int check_launch(const char* what) {
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return fail(SNNF_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(err));
    return SNNF_OK;
}

inline bool valid_dtype(int dt) { return dt == SNNF_F32 || dt == SNNF_BF16 || dt == SNNF_F16; }
inline int dtype_size(int dt) { return dt == SNNF_F32 ? 4 : 2; }
// Compute units of the current device (256 when it cannot be queried).
inline int compute_units() {
    static int cached = 0;
    if (cached == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            cached = n;
        else
            cached = 256;
    }
    return cached;
}

inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// ---------------------------------------------------------------------------------------------------------------
// Storage types. 16-bit floats travel as raw bit patterns; arithmetic is always fp32.
// ---------------------------------------------------------------------------------------------------------------
struct bf16_t { uint16_t bits; };
struct f16_t { uint16_t bits; };

template <typename T> struct dtype_of;
template <> struct dtype_of<float> { static constexpr int value = SNNF_F32; };
template <> struct dtype_of<bf16_t> { static constexpr int value = SNNF_BF16; };
template <> struct dtype_of<f16_t> { static constexpr int value = SNNF_F16; };

__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits) { return __uint_as_float(bits << 16); }

// Round-to-nearest-even fp32 -> bf16 (NaN kept quiet), the rounding torch applies in .to(torch.bfloat16).
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

// The bf16 term of an fp32 value for part `part` of the split described at kSplitParts (snnf_conv_common.h): the value
// rounded to bf16 (parts 0 and 1) or what that rounding left over, rounded to bf16 (part 2). x - hi is exact in fp32.
__device__ __forceinline__ uint32_t split_bf16_bits(float x, bool low_term) {
    const uint32_t hi = float_to_bf16_bits(x);
    if (!low_term) return hi;
    return float_to_bf16_bits(x - __uint_as_float(hi << 16));
}

__device__ __forceinline__ float f16_bits_to_float(uint32_t bits) {
    union { uint16_t u; _Float16 h; } cvt;
    cvt.u = static_cast<uint16_t>(bits);
    return static_cast<float>(cvt.h);
}

__device__ __forceinline__ uint32_t float_to_f16_bits(float f) {
    union { uint16_t u; _Float16 h; } cvt;
    cvt.h = static_cast<_Float16>(f);
    return cvt.u;
}

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return bf16_bits_to_float(v.bits); }
__device__ __forceinline__ float to_float(f16_t v) { return f16_bits_to_float(v.bits); }

template <typename T> __device__ __forceinline__ T from_float(float f);
template <> __device__ __forceinline__ float from_float<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float f) {
    return bf16_t{static_cast<uint16_t>(float_to_bf16_bits(f))};
}
template <> __device__ __forceinline__ f16_t from_float<f16_t>(float f) {
    return f16_t{static_cast<uint16_t>(float_to_f16_bits(f))};
}

// 0/1 spike in storage type T.
template <typename T> __device__ __forceinline__ T spike_value(bool fired);
template <> __device__ __forceinline__ float spike_value<float>(bool fired) { return fired ? 1.0f : 0.0f; }
template <> __device__ __forceinline__ bf16_t spike_value<bf16_t>(bool fired) {
    return bf16_t{static_cast<uint16_t>(fired ? 0x3f80u : 0u)};
}
template <> __device__ __forceinline__ f16_t spike_value<f16_t>(bool fired) {
    return f16_t{static_cast<uint16_t>(fired ? 0x3c00u : 0u)};
}

// N consecutive elements of T moved as one naturally aligned vector.
template <typename T, int N> struct alignas(sizeof(T) * N > 16 ? 16 : sizeof(T) * N) Pack { T v[N]; };

// Store of results that this kernel does not read again (spikes, final membranes): marked non-temporal, so that the
// lines stream through L2 instead of displacing the operands that are re-read (on the MobileNet pointwise layer the
// same stores without the mark cost 17 % of the kernel's time). Used for launches whose outputs exceed what the caches
// hold; smaller outputs are stored normally and stay cached for the kernel that reads them. `dst` is aligned like the pack.
constexpr int64_t kStreamOutBytes = 64ll << 20;   // outputs of a launch from which on they are stored non-temporally (twice the L2s)
typedef uint32_t snnf_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t snnf_u32x2 __attribute__((ext_vector_type(2)));
template <typename T, int N>
__device__ __forceinline__ void store_streaming(T* dst, const Pack<T, N>& value) {
    constexpr int kBytes = static_cast<int>(sizeof(T)) * N;
    // The empty statements keep these stores apart from an ordinary store of the same value on the other side of a
    // branch: merged, the two would become one store without the mark.
    asm volatile("");
    if constexpr (kBytes % 16 == 0) {
#pragma unroll
        for (int i = 0; i < kBytes / 16; ++i)
            __builtin_nontemporal_store(reinterpret_cast<const snnf_u32x4*>(&value)[i], reinterpret_cast<snnf_u32x4*>(dst) + i);
    } else if constexpr (kBytes == 8) {
        __builtin_nontemporal_store(*reinterpret_cast<const snnf_u32x2*>(&value), reinterpret_cast<snnf_u32x2*>(dst));
    } else if constexpr (kBytes == 4) {
        __builtin_nontemporal_store(*reinterpret_cast<const uint32_t*>(&value), reinterpret_cast<uint32_t*>(dst));
    } else {
        *reinterpret_cast<Pack<T, N>*>(dst) = value;
    }
    asm volatile("");
}

// ---------------------------------------------------------------------------------------------------------------
// LIF neuron (runtime/snn_custom_ops.py:384-409). The charge rule is chosen on the host once per launch.
// ---------------------------------------------------------------------------------------------------------------
enum ChargeMode : int {
    CHARGE_IF = 0,        // tau <= 1:            h = v + x
    CHARGE_SCALE = 1,     // tau a power of two:  h = v + (x - v) * (1 / tau)   (bit-identical to the division)
    CHARGE_DIVIDE = 2     // any other tau:       h = v + (x - v) / tau
};

struct LifParams {
    float v_threshold;
    float v_reset;
    float tau;
    float inv_tau;
    int charge_mode;
    int soft_reset;  // v_reset < 0
};

inline LifParams make_lif_params(float v_threshold, float v_reset, float tau) {
    LifParams p;
    p.v_threshold = v_threshold;
    p.v_reset = v_reset;
    p.tau = tau;
    p.inv_tau = 1.0f;
    p.soft_reset = v_reset < 0.0f ? 1 : 0;
    if (tau <= 1.0f) {
        p.charge_mode = CHARGE_IF;
    } else {
        uint32_t bits;
        static_assert(sizeof(bits) == sizeof(tau), "float is 32 bit");
        __builtin_memcpy(&bits, &tau, sizeof(bits));
        const bool pow2 = (bits & 0x007fffffu) == 0u && ((bits >> 23) & 0xffu) != 0u && ((bits >> 23) & 0xffu) < 0xfeu;
        p.charge_mode = pow2 ? CHARGE_SCALE : CHARGE_DIVIDE;
        p.inv_tau = 1.0f / tau;
    }
    return p;
}

// One LIF step: updates v in place, returns whether the neuron fired.
__device__ __forceinline__ bool lif_step(float x, float& v, const LifParams& p) {
    float h;
    if (p.charge_mode == CHARGE_IF) {
        h = v + x;
    } else if (p.charge_mode == CHARGE_SCALE) {
        h = v + (x - v) * p.inv_tau;
    } else {
        h = v + __fdiv_rn(x - v, p.tau);
    }
    const bool fired = h >= p.v_threshold;
    if (p.soft_reset) {
        v = fired ? h - p.v_threshold : h;
    } else {
        v = fired ? p.v_reset : h;
    }
    return fired;
}

// Up to SNNF_MAX_T_PER_LAUNCH per-timestep base pointers, passed to kernels by value.
struct StepPtrs {
    const void* p[SNNF_MAX_T_PER_LAUNCH];
};

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace snnf
