// Repacks an OIHW convolution weight (+ bias) into the fragment order the implicit-GEMM kernel reads.
#include <algorithm>

#include "snnf_conv_common.h"

namespace snnf {
namespace {

template <typename WT, bool TO_F16>
__global__ void pack_weight_kernel(const WT* __restrict__ w, const WT* __restrict__ bias, PackGeom p,
                                   uint16_t* __restrict__ packed, float* __restrict__ bias_out) {
    const int64_t total = static_cast<int64_t>(packed_weight_elems(p));
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx < total) {
        const int j = idx & 7;
        const int lane = (idx >> 3) & 63;
        int64_t frag = idx >> 9;
        const int pair = frag % p.npairs;
        frag /= p.npairs;
        const int vchunk = frag % p.nchunks;
        const int ocf = frag / p.nchunks;
        // fp32 tensors: three parts of the channel axis hold w_hi, w_lo, w_hi (see kSplitParts).
        const int part = vchunk / p.nchunks_r;
        const int chunk = vchunk - part * p.nchunks_r;
        const int oc = ocf * 32 + (lane & 31);
        const int slot = pair * 2 + (lane >> 5);
        const int groups = p.CK / 8;
        const int tap = slot / groups;
        const int ci = chunk * p.CK + (slot % groups) * 8 + j;
        float v = 0.0f;
        if (oc < p.Cout && ci < p.Cin && tap < p.KH * p.KW)
            v = to_float(w[(static_cast<int64_t>(oc) * p.Cin + ci) * (p.KH * p.KW) + tap]);
        packed[idx] = TO_F16 ? static_cast<uint16_t>(float_to_f16_bits(v)) : static_cast<uint16_t>(split_bf16_bits(v, part == 1));
    }
    if (idx < static_cast<int64_t>(packed_bias_floats(p))) bias_out[idx] = (bias != nullptr && idx < p.Cout) ? to_float(bias[idx]) : 0.0f;
}

}  // namespace
}  // namespace snnf

extern "C" size_t snnf_conv_packed_weight_bytes(int Cout, int Cin, int KH, int KW, int x_dtype) {
    using namespace snnf;
    if (Cout < 1 || Cin < 1 || KH < 1 || KW < 1 || !valid_dtype(x_dtype)) return 0;
    const PackGeom p = make_pack_geom(Cout, Cin, KH, KW, x_dtype == SNNF_F32);
    return packed_weight_elems(p) * 2 + packed_bias_floats(p) * sizeof(float);
}

extern "C" int snnf_conv_pack_weight(const void* weight, const void* bias, int w_dtype, int Cout, int Cin, int KH, int KW,
                                     int x_dtype, void* packed, size_t packed_bytes, void* stream) {
    using namespace snnf;
    if (weight == nullptr || packed == nullptr)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_pack_weight: weight and packed must be non-null");
    if (Cout < 1 || Cin < 1 || KH < 1 || KW < 1)
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_pack_weight: Cout=%d Cin=%d KH=%d KW=%d", Cout, Cin, KH, KW);
    if (!valid_dtype(w_dtype) || !valid_dtype(x_dtype))
        return fail(SNNF_ERR_INVALID_ARGUMENT, "snnf_conv_pack_weight: unknown dtype code");
    const size_t need = snnf_conv_packed_weight_bytes(Cout, Cin, KH, KW, x_dtype);
    if (packed_bytes < need || !aligned_to(packed, 16))
        return fail(SNNF_ERR_WORKSPACE, "snnf_conv_pack_weight: packed buffer needs %zu bytes, 16-byte aligned", need);
    const PackGeom p = make_pack_geom(Cout, Cin, KH, KW, x_dtype == SNNF_F32);
    const int64_t total = static_cast<int64_t>(packed_weight_elems(p));
    uint16_t* out = static_cast<uint16_t*>(packed);
    float* bias_out = reinterpret_cast<float*>(out + total);
    const unsigned blocks = static_cast<unsigned>((std::max<int64_t>(total, static_cast<int64_t>(packed_bias_floats(p))) + 255) / 256);
    hipStream_t hs = as_stream(stream);
    const bool to_f16 = x_dtype == SNNF_F16;
#define SNNF_PACK(WT)                                                                                                   \
    do {                                                                                                                \
        if (to_f16)                                                                                                     \
            pack_weight_kernel<WT, true><<<dim3(blocks), 256, 0, hs>>>(static_cast<const WT*>(weight),                 \
                                                                       static_cast<const WT*>(bias), p, out, bias_out); \
        else                                                                                                            \
            pack_weight_kernel<WT, false><<<dim3(blocks), 256, 0, hs>>>(static_cast<const WT*>(weight),                \
                                                                        static_cast<const WT*>(bias), p, out, bias_out); \
    } while (0)
    if (w_dtype == SNNF_F32) SNNF_PACK(float);
    else if (w_dtype == SNNF_BF16) SNNF_PACK(bf16_t);
    else SNNF_PACK(f16_t);
#undef SNNF_PACK
    return check_launch("snnf_conv_pack_weight");
}
