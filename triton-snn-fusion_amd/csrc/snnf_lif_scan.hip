// Temporal LIF scan: streams x[t] once, keeps the membrane in registers for all T steps, writes dense 0/1 spikes
// once and the final membrane once. Bound by HBM bandwidth: (2*T + 1) * numel elements of traffic, ~6 flops each.
#include "snnf_common.h"

namespace snnf {
namespace {

constexpr int kThreads = 256;

// One thread owns VEC consecutive neurons; every load/store of a thread is one 16-byte (or narrower, VEC == 1)
// transaction, so a 64-lane wave moves 1 KiB per instruction.
template <typename XT, typename VT, int VEC, int TC>
__global__ __launch_bounds__(kThreads) void lif_scan_kernel(StepPtrs xs, int T, int64_t numel,
                                                            const VT* __restrict__ v_init, XT* __restrict__ spikes,
                                                            int64_t spike_step_stride, VT* __restrict__ v_out,
                                                            LifParams lif) {
    const int64_t first = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) * VEC;
    if (first >= numel) return;
    using XV = Pack<XT, VEC>;
    using VV = Pack<VT, VEC>;

    float v[VEC];
    if (v_init != nullptr) {
        const VV vi = *reinterpret_cast<const VV*>(v_init + first);
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = to_float(vi.v[i]);
    } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = 0.0f;
    }

    const int steps = TC > 0 ? TC : T;
    if constexpr (TC > 0) {
        // Issue every timestep's load before the recurrence so that T independent 16-byte loads are in flight.
        XV xin[TC];
#pragma unroll
        for (int t = 0; t < TC; ++t) xin[t] = *reinterpret_cast<const XV*>(static_cast<const XT*>(xs.p[t]) + first);
#pragma unroll
        for (int t = 0; t < TC; ++t) {
            XV out;
#pragma unroll
            for (int i = 0; i < VEC; ++i) out.v[i] = spike_value<XT>(lif_step(to_float(xin[t].v[i]), v[i], lif));
            *reinterpret_cast<XV*>(spikes + t * spike_step_stride + first) = out;
        }
    } else {
        for (int t = 0; t < steps; ++t) {
            const XV xin = *reinterpret_cast<const XV*>(static_cast<const XT*>(xs.p[t]) + first);
            XV out;
#pragma unroll
            for (int i = 0; i < VEC; ++i) out.v[i] = spike_value<XT>(lif_step(to_float(xin.v[i]), v[i], lif));
            *reinterpret_cast<XV*>(spikes + t * spike_step_stride + first) = out;
        }
    }

    VV vo;
#pragma unroll
    for (int i = 0; i < VEC; ++i) vo.v[i] = from_float<VT>(v[i]);
    *reinterpret_cast<VV*>(v_out + first) = vo;
}

template <typename XT, typename VT, int VEC>
int launch_lif_scan(const StepPtrs& xs, int T, int64_t numel, const void* v_init, void* spikes,
                    int64_t spike_step_stride, void* v_out, const LifParams& lif, hipStream_t stream) {
    const int64_t threads = (numel + VEC - 1) / VEC;
    const int64_t blocks = (threads + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffffLL) return fail(SNNF_ERR_UNSUPPORTED, "snnf_lif_scan: numel %lld too large", (long long)numel);
    const dim3 grid(static_cast<unsigned>(blocks));
    const VT* vi = static_cast<const VT*>(v_init);
    XT* sp = static_cast<XT*>(spikes);
    VT* vo = static_cast<VT*>(v_out);
    switch (T) {
        case 1: lif_scan_kernel<XT, VT, VEC, 1><<<grid, kThreads, 0, stream>>>(xs, T, numel, vi, sp, spike_step_stride, vo, lif); break;
        case 2: lif_scan_kernel<XT, VT, VEC, 2><<<grid, kThreads, 0, stream>>>(xs, T, numel, vi, sp, spike_step_stride, vo, lif); break;
        case 4: lif_scan_kernel<XT, VT, VEC, 4><<<grid, kThreads, 0, stream>>>(xs, T, numel, vi, sp, spike_step_stride, vo, lif); break;
        case 8: lif_scan_kernel<XT, VT, VEC, 8><<<grid, kThreads, 0, stream>>>(xs, T, numel, vi, sp, spike_step_stride, vo, lif); break;
        default: lif_scan_kernel<XT, VT, VEC, 0><<<grid, kThreads, 0, stream>>>(xs, T, numel, vi, sp, spike_step_stride, vo, lif); break;
    }
    return check_launch("snnf_lif_scan");
}

template <typename XT, typename VT>
int dispatch_vec(bool wide, const StepPtrs& xs, int T, int64_t numel, const void* v_init, void* spikes,
                 int64_t spike_step_stride, void* v_out, const LifParams& lif, hipStream_t stream) {
    constexpr int kWide = 16 / sizeof(XT);
    if (wide) return launch_lif_scan<XT, VT, kWide>(xs, T, numel, v_init, spikes, spike_step_stride, v_out, lif, stream);
    return launch_lif_scan<XT, VT, 1>(xs, T, numel, v_init, spikes, spike_step_stride, v_out, lif, stream);
}

}  // namespace
}  // namespace snnf

extern "C" int snnf_lif_scan(const void* const* xs, int T, int64_t numel, int x_dtype, const void* v_init, int v_dtype,
                             void* spikes, int64_t spike_step_stride, void* v_out, float v_threshold, float v_reset,
                             float tau, void* stream) {
    using namespace snnf;
    if (xs == nullptr || spikes == nullptr || v_out == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_lif_scan: xs, spikes and v_out must be non-null");
    if (T < 1 || numel < 0) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_lif_scan: T=%d numel=%lld", T, (long long)numel);
    if (!valid_dtype(x_dtype) || !valid_dtype(v_dtype))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_lif_scan: unknown dtype code x=%d v=%d", x_dtype, v_dtype);
    if (v_dtype != SNNF_F32 && v_dtype != x_dtype)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_lif_scan: membrane dtype must be fp32 or the activation dtype");
    if (!(tau != 0.0f)) return fail(SNNF_ERR_UNSUPPORTED, "snnf_lif_scan: unsupported_tau: tau must be nonzero");
    for (int t = 0; t < T; ++t)
        if (xs[t] == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_lif_scan: xs[%d] is null", t);
    if (numel == 0) return SNNF_OK;

    const LifParams lif = make_lif_params(v_threshold, v_reset, tau);
    const int xsize = dtype_size(x_dtype);
    const int per_vec = 16 / xsize;
    const size_t v_align = static_cast<size_t>(per_vec) * dtype_size(v_dtype);
    hipStream_t hs = as_stream(stream);

    // Windows of at most SNNF_MAX_T_PER_LAUNCH steps; later windows continue from v_out in place.
    for (int t0 = 0; t0 < T; t0 += SNNF_MAX_T_PER_LAUNCH) {
        const int tw = (T - t0) < SNNF_MAX_T_PER_LAUNCH ? (T - t0) : SNNF_MAX_T_PER_LAUNCH;
        StepPtrs ptrs = {};
        bool wide = (numel % per_vec) == 0 && (spike_step_stride % per_vec) == 0 && aligned_to(spikes, 16) &&
                    aligned_to(v_out, v_align > 16 ? 16 : v_align);
        for (int t = 0; t < tw; ++t) {
            ptrs.p[t] = xs[t0 + t];
            wide = wide && aligned_to(xs[t0 + t], 16);
        }
        const void* vi = t0 == 0 ? v_init : v_out;
        if (vi != nullptr) wide = wide && aligned_to(vi, v_align > 16 ? 16 : v_align);
        void* sp = static_cast<char*>(spikes) + static_cast<int64_t>(t0) * spike_step_stride * xsize;

        int rc;
        if (x_dtype == SNNF_F32) {
            rc = dispatch_vec<float, float>(wide, ptrs, tw, numel, vi, sp, spike_step_stride, v_out, lif, hs);
        } else if (x_dtype == SNNF_BF16) {
            rc = v_dtype == SNNF_F32
                     ? dispatch_vec<bf16_t, float>(wide, ptrs, tw, numel, vi, sp, spike_step_stride, v_out, lif, hs)
                     : dispatch_vec<bf16_t, bf16_t>(wide, ptrs, tw, numel, vi, sp, spike_step_stride, v_out, lif, hs);
        } else {
            rc = v_dtype == SNNF_F32
                     ? dispatch_vec<f16_t, float>(wide, ptrs, tw, numel, vi, sp, spike_step_stride, v_out, lif, hs)
                     : dispatch_vec<f16_t, f16_t>(wide, ptrs, tw, numel, vi, sp, spike_step_stride, v_out, lif, hs);
        }
        if (rc != SNNF_OK) return rc;
    }
    return SNNF_OK;
}
