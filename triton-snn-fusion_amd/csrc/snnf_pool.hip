// 2-D max / average pooling over NCHW planes of spikes (or any activations): the stateless layer between fused operators
// in a spiking CNN (3x3/2 max pool after a ResNet stem, 2x2 average pools between VGG stages). Bound by HBM bandwidth:
// every input element is read once from memory (neighbouring windows re-read it from cache), every output written once.
#include "snnf_common.h"

namespace snnf {
namespace {

constexpr int kThreads = 256;
constexpr int kOutPerThread = 4;   // consecutive outputs of one output row per thread

// One thread produces up to 4 consecutive outputs of an output row; a wave covers 256 consecutive outputs, so its loads
// walk consecutive input addresses row by row. Average pooling divides by K * K (padding is not allowed for it).
template <typename XT, int K, int S, bool IS_MAX>
__global__ __launch_bounds__(kThreads) void pool2d_kernel(const XT* __restrict__ x, XT* __restrict__ y, int64_t planes,
                                                          int H, int W, int Ho, int Wo, int pad, int strips_per_row) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int64_t rows = planes * Ho;
    const int64_t row = item / strips_per_row;
    if (row >= rows) return;
    const int ox0 = static_cast<int>(item - row * strips_per_row) * kOutPerThread;
    const int64_t plane = row / Ho;
    const int oy = static_cast<int>(row - plane * Ho);
    const XT* __restrict__ src = x + plane * H * W;
    float acc[kOutPerThread];
#pragma unroll
    for (int j = 0; j < kOutPerThread; ++j) acc[j] = IS_MAX ? -3.0e38f : 0.0f;
    constexpr int SPAN = (kOutPerThread - 1) * S + K;   // input columns under the strip
#pragma unroll
    for (int ky = 0; ky < K; ++ky) {
        const int iy = oy * S - pad + ky;
        if (iy < 0 || iy >= H) continue;
        float v[SPAN];
#pragma unroll
        for (int c = 0; c < SPAN; ++c) {
            const int ix = ox0 * S - pad + c;
            v[c] = (ix >= 0 && ix < W) ? to_float(src[static_cast<int64_t>(iy) * W + ix]) : (IS_MAX ? -3.0e38f : 0.0f);
        }
#pragma unroll
        for (int j = 0; j < kOutPerThread; ++j)
#pragma unroll
            for (int kx = 0; kx < K; ++kx) acc[j] = IS_MAX ? fmaxf(acc[j], v[j * S + kx]) : acc[j] + v[j * S + kx];
    }
    XT* __restrict__ dst = y + (plane * Ho + oy) * Wo + ox0;
#pragma unroll
    for (int j = 0; j < kOutPerThread; ++j)
        if (ox0 + j < Wo) dst[j] = from_float<XT>(IS_MAX ? acc[j] : acc[j] * (1.0f / (K * K)));
}

// Stride-2 pooling of 16-bit planes whose rows are whole 16-byte groups (W % 8 == 0, aligned base): the 8 input columns
// under a thread's 4 outputs arrive in one 16-byte load per row (plus the single column to their left for a padded 3x3
// window), the 4 outputs leave in one 8-byte store.
template <typename XT, int K, bool IS_MAX>
__global__ __launch_bounds__(kThreads) void pool2d_s2_vec_kernel(const XT* __restrict__ x, XT* __restrict__ y, int64_t planes,
                                                                 int H, int W, int Ho, int Wo, int strips_per_row) {
    static_assert(sizeof(XT) == 2 && (K == 2 || K == 3), "16-bit activations, 2x2 (no padding) or 3x3 (padding 1) windows");
    constexpr int PAD = K == 3 ? 1 : 0;
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int64_t rows = planes * Ho;
    const int64_t row = item / strips_per_row;
    if (row >= rows) return;
    const int ox0 = static_cast<int>(item - row * strips_per_row) * 4;
    const int64_t plane = row / Ho;
    const int oy = static_cast<int>(row - plane * Ho);
    const XT* __restrict__ src = x + plane * H * W + 2 * ox0;
    float acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = IS_MAX ? -3.0e38f : 0.0f;
#pragma unroll
    for (int ky = 0; ky < K; ++ky) {
        // No branch around a load (the compiler would wait for each load before issuing the next): a window row outside
        // the plane re-reads the nearest row inside, which belongs to the same window and leaves a maximum unchanged
        // (unpadded 2x2 windows never leave the plane); the column left of the first one re-reads the first.
        const int iy = min(max(oy * 2 - PAD + ky, 0), H - 1);
        const XT* __restrict__ line = src + static_cast<int64_t>(iy) * W;
        const Pack<XT, 8> eight = *reinterpret_cast<const Pack<XT, 8>*>(line);
        float v[9];
#pragma unroll
        for (int c = 0; c < 8; ++c) v[1 + c] = to_float(eight.v[c]);
        if constexpr (PAD == 1) {
            const float left = to_float(line[ox0 > 0 ? -1 : 0]);
            v[0] = ox0 > 0 ? left : -3.0e38f;
        } else {
            v[0] = -3.0e38f;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (K == 3) acc[j] = fmaxf(fmaxf(acc[j], v[2 * j]), fmaxf(v[2 * j + 1], v[2 * j + 2]));
            else acc[j] = IS_MAX ? fmaxf(acc[j], fmaxf(v[1 + 2 * j], v[2 + 2 * j])) : acc[j] + v[1 + 2 * j] + v[2 + 2 * j];
        }
    }
    Pack<XT, 4> out;
#pragma unroll
    for (int j = 0; j < 4; ++j) out.v[j] = from_float<XT>((IS_MAX || K == 3) ? acc[j] : acc[j] * 0.25f);
    *reinterpret_cast<Pack<XT, 4>*>(y + (plane * Ho + oy) * Wo + ox0) = out;
}

template <typename XT>
int launch_pool(const void* x, void* y, int64_t planes, int H, int W, int k, int stride, int pad, int is_max, hipStream_t stream) {
    const int Ho = (H + 2 * pad - k) / stride + 1;
    const int Wo = (W + 2 * pad - k) / stride + 1;
    const int strips = (Wo + kOutPerThread - 1) / kOutPerThread;
    const int64_t items = planes * Ho * strips;
    const int64_t blocks = (items + kThreads - 1) / kThreads;
    if (blocks > 0x7fffffff) return fail(SNNF_ERR_UNSUPPORTED, "snnf_pool2d: unsupported_shape: too many outputs");
    const dim3 grid(static_cast<unsigned>(blocks));
    const XT* xs = static_cast<const XT*>(x);
    XT* ys = static_cast<XT*>(y);
    if constexpr (sizeof(XT) == 2) {
        const bool rows_vectorize = stride == 2 && W % 8 == 0 && aligned_to(x, 16) && aligned_to(y, 8);
        if (rows_vectorize && is_max && k == 3 && pad == 1) {
            pool2d_s2_vec_kernel<XT, 3, true><<<grid, kThreads, 0, stream>>>(xs, ys, planes, H, W, Ho, Wo, strips);
            return check_launch("snnf_pool2d");
        }
        if (rows_vectorize && k == 2 && pad == 0) {
            if (is_max) pool2d_s2_vec_kernel<XT, 2, true><<<grid, kThreads, 0, stream>>>(xs, ys, planes, H, W, Ho, Wo, strips);
            else pool2d_s2_vec_kernel<XT, 2, false><<<grid, kThreads, 0, stream>>>(xs, ys, planes, H, W, Ho, Wo, strips);
            return check_launch("snnf_pool2d");
        }
    }
    if (is_max && k == 3 && stride == 2) pool2d_kernel<XT, 3, 2, true><<<grid, kThreads, 0, stream>>>(xs, ys, planes, H, W, Ho, Wo, pad, strips);
    else if (is_max && k == 2 && stride == 2) pool2d_kernel<XT, 2, 2, true><<<grid, kThreads, 0, stream>>>(xs, ys, planes, H, W, Ho, Wo, pad, strips);
    else if (!is_max && k == 2 && stride == 2) pool2d_kernel<XT, 2, 2, false><<<grid, kThreads, 0, stream>>>(xs, ys, planes, H, W, Ho, Wo, pad, strips);
    else return fail(SNNF_ERR_UNSUPPORTED, "snnf_pool2d: unsupported_kernel: max 3x3/2, max 2x2/2 and average 2x2/2 are implemented, got %s %dx%d/%d",
                     is_max ? "max" : "average", k, k, stride);
    return check_launch("snnf_pool2d");
}

}  // namespace
}  // namespace snnf

extern "C" int snnf_pool2d(const void* x, void* y, int64_t planes, int H, int W, int kernel, int stride, int pad, int is_max,
                           int x_dtype, void* stream) {
    using namespace snnf;
    if (x == nullptr || y == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_pool2d: x and y must be non-null");
    if (planes < 1 || H < 1 || W < 1 || kernel < 1 || stride < 1 || pad < 0)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_pool2d: bad extent (planes=%lld H=%d W=%d k=%d s=%d p=%d)",
                    static_cast<long long>(planes), H, W, kernel, stride, pad);
    if (!valid_dtype(x_dtype)) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_pool2d: unknown dtype code");
    if (2 * pad > kernel || (!is_max && pad != 0))
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_pool2d: unsupported_padding: padding %d for a %s pool of size %d", pad, is_max ? "max" : "average", kernel);
    if (H + 2 * pad < kernel || W + 2 * pad < kernel) return fail(SNNF_ERR_UNSUPPORTED, "snnf_pool2d: unsupported_kernel: window larger than the padded plane");
    hipStream_t hs = static_cast<hipStream_t>(stream);
    if (x_dtype == SNNF_F32) return launch_pool<float>(x, y, planes, H, W, kernel, stride, pad, is_max, hs);
    if (x_dtype == SNNF_BF16) return launch_pool<bf16_t>(x, y, planes, H, W, kernel, stride, pad, is_max, hs);
    return launch_pool<f16_t>(x, y, planes, H, W, kernel, stride, pad, is_max, hs);
}
