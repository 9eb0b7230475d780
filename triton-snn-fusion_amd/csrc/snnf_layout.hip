// Internal activation layouts between consecutive fused operators: conversion between dense NCHW, channel-blocked C8
// ([N][C/8][H][W][8] 16-bit elements) and bit-packed BITS ([N][C/8][H][W] bytes, bit j = channel 8 c8 + j), and 2-D pooling
// on the two internal layouts. All of it is bound by HBM bandwidth; a thread owns one group of 8 channels of one pixel, so
// the threads of a wave walk consecutive pixels (coalesced in every layout).
#include "snnf_common.h"

namespace snnf {
namespace {

constexpr int kThreads = 256;

// The 8 channels of group c8 at pixel `px` of frame n, as floats (absent channels read as 0).
template <typename XT, int LAYOUT>
__device__ __forceinline__ void load_group(const void* __restrict__ src, int64_t n, int c8, int64_t px, int C, int C8, int64_t HW, float (&v)[8]) {
    if constexpr (LAYOUT == SNNF_LAYOUT_NCHW) {
        const XT* __restrict__ p = static_cast<const XT*>(src) + (n * C + c8 * 8) * HW + px;
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = c8 * 8 + j < C ? to_float(p[j * HW]) : 0.0f;
    } else if constexpr (LAYOUT == SNNF_LAYOUT_C8) {
        const Pack<XT, 8> g = *reinterpret_cast<const Pack<XT, 8>*>(static_cast<const XT*>(src) + ((n * C8 + c8) * HW + px) * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = to_float(g.v[j]);
    } else {
        const uint32_t byte = static_cast<const unsigned char*>(src)[(n * C8 + c8) * HW + px];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = ((byte >> j) & 1u) ? 1.0f : 0.0f;
    }
}

template <typename XT, int LAYOUT>
__device__ __forceinline__ void store_group(void* __restrict__ dst, int64_t n, int c8, int64_t px, int C, int C8, int64_t HW, const float (&v)[8]) {
    if constexpr (LAYOUT == SNNF_LAYOUT_NCHW) {
        XT* __restrict__ p = static_cast<XT*>(dst) + (n * C + c8 * 8) * HW + px;
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (c8 * 8 + j < C) p[j * HW] = from_float<XT>(v[j]);
    } else if constexpr (LAYOUT == SNNF_LAYOUT_C8) {
        Pack<XT, 8> g;
#pragma unroll
        for (int j = 0; j < 8; ++j) g.v[j] = from_float<XT>(c8 * 8 + j < C ? v[j] : 0.0f);
        *reinterpret_cast<Pack<XT, 8>*>(static_cast<XT*>(dst) + ((n * C8 + c8) * HW + px) * 8) = g;
    } else {
        uint32_t byte = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) byte |= (c8 * 8 + j < C && v[j] != 0.0f) ? (1u << j) : 0u;
        static_cast<unsigned char*>(dst)[(n * C8 + c8) * HW + px] = static_cast<unsigned char>(byte);
    }
}

template <typename XT, int SRC, int DST>
__global__ __launch_bounds__(kThreads) void layout_convert_kernel(const void* __restrict__ src, void* __restrict__ dst, int64_t frames,
                                                                  int C, int C8, int64_t HW) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (item >= frames * C8 * HW) return;
    const int64_t plane = item / HW;
    const int64_t px = item - plane * HW;
    const int64_t n = plane / C8;
    const int c8 = static_cast<int>(plane - n * C8);
    float v[8];
    load_group<XT, SRC>(src, n, c8, px, C, C8, HW, v);
    store_group<XT, DST>(dst, n, c8, px, C, C8, HW, v);
}

// Pooling of one group of 8 channels per thread: K x K window, stride 2, `pad` rows/columns of padding that never win a
// maximum (average pooling takes no padding). Spikes are 0 / 1, so a maximum over bits is their OR.
template <typename XT, int SRC, int DST, int K, bool IS_MAX>
__global__ __launch_bounds__(kThreads) void pool_blocked_kernel(const void* __restrict__ x, void* __restrict__ y, int64_t frames, int C, int C8,
                                                                int H, int W, int Ho, int Wo, int pad) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int64_t HWo = static_cast<int64_t>(Ho) * Wo;
    if (item >= frames * C8 * HWo) return;
    const int64_t plane = item / HWo;
    const int po = static_cast<int>(item - plane * HWo);
    const int64_t n = plane / C8;
    const int c8 = static_cast<int>(plane - n * C8);
    const int oy = po / Wo, ox = po - oy * Wo;
    const int64_t HW = static_cast<int64_t>(H) * W;
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = IS_MAX ? -3.0e38f : 0.0f;
    uint32_t bits = 0;
#pragma unroll
    for (int ky = 0; ky < K; ++ky) {
        const int iy = oy * 2 - pad + ky;
        if (iy < 0 || iy >= H) continue;
#pragma unroll
        for (int kx = 0; kx < K; ++kx) {
            const int ix = ox * 2 - pad + kx;
            if (ix < 0 || ix >= W) continue;
            if constexpr (SRC == SNNF_LAYOUT_BITS && IS_MAX) {
                bits |= static_cast<const unsigned char*>(x)[(n * C8 + c8) * HW + static_cast<int64_t>(iy) * W + ix];
            } else {
                float v[8];
                load_group<XT, SRC>(x, n, c8, static_cast<int64_t>(iy) * W + ix, C, C8, HW, v);
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] = IS_MAX ? fmaxf(acc[j], v[j]) : acc[j] + v[j];
            }
        }
    }
    if constexpr (SRC == SNNF_LAYOUT_BITS && IS_MAX) {
        static_cast<unsigned char*>(y)[(n * C8 + c8) * HWo + po] = static_cast<unsigned char>(bits);
    } else {
        if constexpr (!IS_MAX) {
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] *= 1.0f / (K * K);
        }
        store_group<XT, DST>(y, n, c8, po, C, C8, HWo, acc);
    }
}

// Maximum pooling of bit-packed spikes, four neighbouring output pixels of one channel group per thread, for rows whose
// bytes can be taken eight at a time (W % 8 == 0, Wo == W / 2, a 16-byte aligned tensor is not needed: planes are multiples
// of 8 bytes from an 8-byte aligned base). The OR of a window's bytes lands in the even bytes of the row word; K == 3 has
// one column of padding on the left, which is the byte in front of the word (absent at the row's start).
template <int K>
__global__ __launch_bounds__(kThreads) void pool_bits_rows_kernel(const unsigned char* __restrict__ x, uint32_t* __restrict__ y, int64_t planes,
                                                                  int H, int W, int Ho, int Wq) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int64_t per_plane = static_cast<int64_t>(Ho) * Wq;
    if (item >= planes * per_plane) return;
    const int64_t plane = item / per_plane;
    const int rem = static_cast<int>(item - plane * per_plane);
    const int oy = rem / Wq, m = rem - oy * Wq;
    const unsigned char* src = x + plane * (static_cast<int64_t>(H) * W) + m * 8;
    constexpr int PAD = K == 3 ? 1 : 0;
    uint64_t acc = 0;
#pragma unroll
    for (int ky = 0; ky < K; ++ky) {
        const int iy = oy * 2 - PAD + ky;
        if (iy < 0 || iy >= H) continue;
        const unsigned char* row = src + static_cast<int64_t>(iy) * W;
        const uint64_t q = *reinterpret_cast<const uint64_t*>(row);
        acc |= q | (q >> 8);
        if constexpr (K == 3) acc |= (q << 8) | (m > 0 ? static_cast<uint64_t>(row[-1]) : 0ull);
    }
    y[item] = __builtin_amdgcn_perm(static_cast<uint32_t>(acc >> 32), static_cast<uint32_t>(acc), 0x06040200u);
}

// Average pooling (2 x 2) of bit-packed spikes into channel-blocked quarters, four neighbouring output pixels of one channel
// group per thread: two 8-byte row words in, 64 contiguous bytes out. A channel's value is a quarter of the number of its
// bits among the window's four bytes; padded channels hold zero bits and come out as zeros.
template <typename XT>
__global__ __launch_bounds__(kThreads) void pool_bits_avg_rows_kernel(const unsigned char* __restrict__ x, XT* __restrict__ y, int64_t planes,
                                                                      int H, int W, int Ho, int Wq) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int64_t per_plane = static_cast<int64_t>(Ho) * Wq;
    if (item >= planes * per_plane) return;
    const int64_t plane = item / per_plane;
    const int rem = static_cast<int>(item - plane * per_plane);
    const int oy = rem / Wq, m = rem - oy * Wq;
    const unsigned char* src = x + plane * (static_cast<int64_t>(H) * W) + static_cast<int64_t>(2 * oy) * W + m * 8;
    const uint64_t q0 = *reinterpret_cast<const uint64_t*>(src);
    const uint64_t q1 = *reinterpret_cast<const uint64_t*>(src + W);
    XT* __restrict__ dst = y + (item * 4) * 8;           // output pixel (plane, oy, 4 m) of [planes][Ho][4 Wq][8]
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t window = static_cast<uint32_t>((q0 >> (16 * j)) & 0xffffu) | (static_cast<uint32_t>((q1 >> (16 * j)) & 0xffffu) << 16);
        Pack<XT, 8> out;
#pragma unroll
        for (int c = 0; c < 8; ++c) out.v[c] = from_float<XT>(0.25f * static_cast<float>(__builtin_popcount(window & (0x01010101u << c))));
        *reinterpret_cast<Pack<XT, 8>*>(dst + j * 8) = out;
    }
}

template <typename XT>
int convert_typed(const void* src, int sl, void* dst, int dl, int64_t frames, int C, int C8, int64_t HW, unsigned blocks, hipStream_t hs) {
#define SNNF_CONVERT(S, D)                                                                                                   \
    if (sl == S && dl == D) {                                                                                               \
        layout_convert_kernel<XT, S, D><<<dim3(blocks), kThreads, 0, hs>>>(src, dst, frames, C, C8, HW);                   \
        return check_launch("snnf_layout_convert");                                                                         \
    }
    SNNF_CONVERT(SNNF_LAYOUT_NCHW, SNNF_LAYOUT_C8)
    SNNF_CONVERT(SNNF_LAYOUT_NCHW, SNNF_LAYOUT_BITS)
    SNNF_CONVERT(SNNF_LAYOUT_C8, SNNF_LAYOUT_NCHW)
    SNNF_CONVERT(SNNF_LAYOUT_C8, SNNF_LAYOUT_BITS)
    SNNF_CONVERT(SNNF_LAYOUT_BITS, SNNF_LAYOUT_NCHW)
    SNNF_CONVERT(SNNF_LAYOUT_BITS, SNNF_LAYOUT_C8)
    SNNF_CONVERT(SNNF_LAYOUT_NCHW, SNNF_LAYOUT_NCHW)
    SNNF_CONVERT(SNNF_LAYOUT_C8, SNNF_LAYOUT_C8)
    SNNF_CONVERT(SNNF_LAYOUT_BITS, SNNF_LAYOUT_BITS)
#undef SNNF_CONVERT
    return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_layout_convert: unknown layout code");
}

template <typename XT>
int pool_typed(const void* x, int xl, void* y, int yl, int64_t frames, int C, int C8, int H, int W, int Ho, int Wo, int kernel, int pad,
               bool is_max, unsigned blocks, hipStream_t hs) {
#define SNNF_POOL(S, D, K, M)                                                                                                \
    if (xl == S && yl == D && kernel == K && is_max == M) {                                                                 \
        pool_blocked_kernel<XT, S, D, K, M><<<dim3(blocks), kThreads, 0, hs>>>(x, y, frames, C, C8, H, W, Ho, Wo, pad);    \
        return check_launch("snnf_pool2d_blocked");                                                                         \
    }
    SNNF_POOL(SNNF_LAYOUT_BITS, SNNF_LAYOUT_BITS, 3, true)
    SNNF_POOL(SNNF_LAYOUT_BITS, SNNF_LAYOUT_BITS, 2, true)
    SNNF_POOL(SNNF_LAYOUT_BITS, SNNF_LAYOUT_C8, 2, false)
    SNNF_POOL(SNNF_LAYOUT_C8, SNNF_LAYOUT_C8, 3, true)
    SNNF_POOL(SNNF_LAYOUT_C8, SNNF_LAYOUT_C8, 2, true)
    SNNF_POOL(SNNF_LAYOUT_C8, SNNF_LAYOUT_C8, 2, false)
#undef SNNF_POOL
    return fail(SNNF_ERR_UNSUPPORTED, "snnf_pool2d_blocked: unsupported_layout: max pooling BITS -> BITS or C8 -> C8, average pooling BITS -> C8 or C8 -> C8");
}

bool known_layout(int l) { return l == SNNF_LAYOUT_NCHW || l == SNNF_LAYOUT_C8 || l == SNNF_LAYOUT_BITS; }

}  // namespace
}  // namespace snnf

extern "C" size_t snnf_layout_bytes(int layout, int64_t frames, int C, int H, int W, int x_dtype) {
    using namespace snnf;
    if (!known_layout(layout) || frames < 1 || C < 1 || H < 1 || W < 1 || !valid_dtype(x_dtype)) return 0;
    const size_t hw = static_cast<size_t>(H) * W;
    const size_t c8 = static_cast<size_t>((C + 7) / 8);
    if (layout == SNNF_LAYOUT_NCHW) return static_cast<size_t>(frames) * C * hw * dtype_size(x_dtype);
    if (layout == SNNF_LAYOUT_C8) return static_cast<size_t>(frames) * c8 * hw * 8 * dtype_size(x_dtype);
    return static_cast<size_t>(frames) * c8 * hw;
}

extern "C" int snnf_layout_convert(const void* src, int src_layout, void* dst, int dst_layout, int64_t frames, int C, int H, int W,
                                   int x_dtype, void* stream) {
    using namespace snnf;
    if (src == nullptr || dst == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_layout_convert: src and dst must be non-null");
    if (frames < 1 || C < 1 || H < 1 || W < 1) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_layout_convert: frames=%lld C=%d H=%d W=%d", (long long)frames, C, H, W);
    if (x_dtype != SNNF_BF16 && x_dtype != SNNF_F16)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_layout_convert: unsupported_dtype: the internal layouts hold bf16 or fp16 activations");
    if (!known_layout(src_layout) || !known_layout(dst_layout)) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_layout_convert: unknown layout code");
    if ((src_layout == SNNF_LAYOUT_C8 && !aligned_to(src, 16)) || (dst_layout == SNNF_LAYOUT_C8 && !aligned_to(dst, 16)))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_layout_convert: C8 tensors must be 16-byte aligned");
    const int C8 = (C + 7) / 8;
    const int64_t HW = static_cast<int64_t>(H) * W;
    const int64_t items = frames * C8 * HW;
    if (items >= (1LL << 40)) return fail(SNNF_ERR_UNSUPPORTED, "snnf_layout_convert: unsupported_shape: too many elements");
    const unsigned blocks = static_cast<unsigned>((items + kThreads - 1) / kThreads);
    hipStream_t hs = as_stream(stream);
    return x_dtype == SNNF_BF16 ? convert_typed<bf16_t>(src, src_layout, dst, dst_layout, frames, C, C8, HW, blocks, hs)
                                : convert_typed<f16_t>(src, src_layout, dst, dst_layout, frames, C, C8, HW, blocks, hs);
}

extern "C" int snnf_pool2d_blocked(const void* x, int x_layout, void* y, int y_layout, int64_t frames, int C, int H, int W, int kernel,
                                   int stride, int pad, int is_max, int x_dtype, void* stream) {
    using namespace snnf;
    if (x == nullptr || y == nullptr) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_pool2d_blocked: x and y must be non-null");
    if (frames < 1 || C < 1 || H < 1 || W < 1) return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_pool2d_blocked: frames=%lld C=%d H=%d W=%d", (long long)frames, C, H, W);
    if (x_dtype != SNNF_BF16 && x_dtype != SNNF_F16)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_pool2d_blocked: unsupported_dtype: the internal layouts hold bf16 or fp16 activations");
    const bool window_ok = stride == 2 && ((is_max && (kernel == 2 || kernel == 3) && pad >= 0 && 2 * pad <= kernel) || (!is_max && kernel == 2 && pad == 0));
    if (!window_ok)
        return fail(SNNF_ERR_UNSUPPORTED, "snnf_pool2d_blocked: unsupported_kernel: max 2x2 / 3x3 stride 2 or average 2x2 stride 2, got %s %dx%d/%d pad %d",
                    is_max ? "max" : "avg", kernel, kernel, stride, pad);
    if (H + 2 * pad < kernel || W + 2 * pad < kernel) return fail(SNNF_ERR_UNSUPPORTED, "snnf_pool2d_blocked: unsupported_kernel: window larger than the padded plane");
    if ((x_layout == SNNF_LAYOUT_C8 && !aligned_to(x, 16)) || (y_layout == SNNF_LAYOUT_C8 && !aligned_to(y, 16)))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_pool2d_blocked: C8 tensors must be 16-byte aligned");
    const int Ho = (H + 2 * pad - kernel) / 2 + 1;
    const int Wo = (W + 2 * pad - kernel) / 2 + 1;
    const int C8 = (C + 7) / 8;
    const int64_t items = frames * C8 * Ho * Wo;
    const unsigned blocks = static_cast<unsigned>((items + kThreads - 1) / kThreads);
    hipStream_t hs = as_stream(stream);
    if (x_layout == SNNF_LAYOUT_BITS && y_layout == SNNF_LAYOUT_BITS && is_max != 0 && W % 8 == 0 && Wo * 2 == W && pad == (kernel == 3 ? 1 : 0) &&
        aligned_to(x, 8) && aligned_to(y, 4)) {
        const int64_t rows = frames * C8 * Ho * (Wo / 4);
        const unsigned row_blocks = static_cast<unsigned>((rows + kThreads - 1) / kThreads);
        if (kernel == 3)
            pool_bits_rows_kernel<3><<<dim3(row_blocks), kThreads, 0, hs>>>(static_cast<const unsigned char*>(x), static_cast<uint32_t*>(y), frames * C8, H, W, Ho, Wo / 4);
        else
            pool_bits_rows_kernel<2><<<dim3(row_blocks), kThreads, 0, hs>>>(static_cast<const unsigned char*>(x), static_cast<uint32_t*>(y), frames * C8, H, W, Ho, Wo / 4);
        return check_launch("snnf_pool2d_blocked");
    }
    if (x_layout == SNNF_LAYOUT_BITS && y_layout == SNNF_LAYOUT_C8 && is_max == 0 && kernel == 2 && pad == 0 && W % 8 == 0 && Wo * 2 == W &&
        aligned_to(x, 8)) {
        const int64_t rows = frames * C8 * Ho * (Wo / 4);
        const unsigned row_blocks = static_cast<unsigned>((rows + kThreads - 1) / kThreads);
        if (x_dtype == SNNF_BF16)
            pool_bits_avg_rows_kernel<bf16_t><<<dim3(row_blocks), kThreads, 0, hs>>>(static_cast<const unsigned char*>(x), static_cast<bf16_t*>(y), frames * C8, H, W, Ho, Wo / 4);
        else
            pool_bits_avg_rows_kernel<f16_t><<<dim3(row_blocks), kThreads, 0, hs>>>(static_cast<const unsigned char*>(x), static_cast<f16_t*>(y), frames * C8, H, W, Ho, Wo / 4);
        return check_launch("snnf_pool2d_blocked");
    }
    return x_dtype == SNNF_BF16 ? pool_typed<bf16_t>(x, x_layout, y, y_layout, frames, C, C8, H, W, Ho, Wo, kernel, pad, is_max != 0, blocks, hs)
                                : pool_typed<f16_t>(x, x_layout, y, y_layout, frames, C, C8, H, W, Ho, Wo, kernel, pad, is_max != 0, blocks, hs);
}
