// Depthwise causal convolution along the token axis (kernel size 2..4, optional bias, SiLU and
// padding mask), with the carry of the last kernel_size - 1 inputs in and out: one kernel for
// prefill, multi-token continuation and the one-token decode update.
//
// Bound: HBM.  Algorithmic bytes per (token, channel): one read of x and one write of y, i.e.
// 2 * sizeof(element); weights, bias, state and mask are negligible.
//
// A thread owns 16 bytes of channels (8 bf16 / 4 fp32) and walks TOKENS consecutive tokens with
// the kernel_size - 1 previous rows in registers, so inside a block every row of x is read once;
// neighbouring token blocks share kernel_size - 1 rows of halo and are walked in opposite directions, so
// that both read them at the same moment.  Lanes cover consecutive channel
// vectors: every load and store of a wave is one contiguous row segment; the four waves of a
// workgroup take consecutive token blocks of the same channels.

#include "gdn_common.h"

namespace gdn {

constexpr int CONV_THREADS = 256;
constexpr int CONV_TOKENS = 16;  // tokens per thread (measured: 16 beats 32, 64, 128; more workgroups in flight)

struct ConvParams {
    const void* x;
    const void* weight;
    const void* bias;
    const void* input_state;
    const void* mask;
    void* y;
    void* final_state;
    int64_t x_stride_b, x_stride_s, y_stride_b, y_stride_s;
    int B, S, C;
};

template <typename T>
struct ConvVec;
template <>
struct ConvVec<bf16_t> {
    static constexpr int N = 8;
    typedef bf16x8 type;
};
template <>
struct ConvVec<float> {
    static constexpr int N = 4;
    typedef f32x4 type;
};

// VEC * KS weights of VEC consecutive channels are contiguous and 16-byte aligned: vector loads
template <typename WT, int N>
__device__ __forceinline__ void load_contiguous(const void* base, int64_t first, float (&out)[N]) {
    constexpr int PER = 16 / sizeof(WT);
    static_assert(N % PER == 0, "whole 16-byte vectors only");
    typedef typename ConvVec<WT>::type wvec_t;
    const wvec_t* src = reinterpret_cast<const wvec_t*>(reinterpret_cast<const WT*>(base) + first);
#pragma unroll
    for (int i = 0; i < N / PER; i++) {
        const wvec_t v = src[i];
#pragma unroll
        for (int e = 0; e < PER; e++) out[i * PER + e] = (float)v[e];
    }
}

template <typename T, typename WT, int KS, bool SILU>
__global__ __launch_bounds__(CONV_THREADS) void causal_conv1d_kernel(const ConvParams p) {
    constexpr int VEC = ConvVec<T>::N;
    typedef typename ConvVec<T>::type vec_t;

    // a workgroup covers 64 channel vectors x (4 waves x CONV_TOKENS tokens): the halo rows of a wave are the
    // last rows of the wave before it, read on the same CU at about the same time
    const int c0 = (blockIdx.x * WAVE + threadIdx.x % WAVE) * VEC;
    if (c0 >= p.C) return;
    const int b = blockIdx.z;
    const int s_begin = (blockIdx.y * (CONV_THREADS / WAVE) + threadIdx.x / WAVE) * CONV_TOKENS;
    if (s_begin >= p.S) return;
    const int s_end = min(s_begin + CONV_TOKENS, p.S);

    const T* xb = reinterpret_cast<const T*>(p.x) + (int64_t)b * p.x_stride_b + c0;
    T* yb = reinterpret_cast<T*>(p.y) + (int64_t)b * p.y_stride_b + c0;
    const T* mb = p.mask == nullptr ? nullptr : reinterpret_cast<const T*>(p.mask) + (int64_t)b * p.S;

    float wflat[VEC * KS], bias[VEC];  // wflat[e * KS + j]: tap j of channel c0 + e
    load_contiguous<WT, VEC * KS>(p.weight, (int64_t)c0 * KS, wflat);
#pragma unroll
    for (int e = 0; e < VEC; e++) bias[e] = 0.f;
    if (p.bias != nullptr) load_contiguous<WT, VEC>(p.bias, c0, bias);

    auto load_row = [&](int s, float (&row)[VEC]) {
        const vec_t v = *reinterpret_cast<const vec_t*>(xb + (int64_t)s * p.x_stride_s);
        const float m = mb == nullptr ? 1.f : (float)mb[s];
#pragma unroll
        for (int e = 0; e < VEC; e++) row[e] = (float)v[e] * m;
    };

    // row s of the (masked) input for s >= 0, the carried state or zeros for the kernel_size - 1 rows before the sequence
    auto load_any = [&](int s, float (&row)[VEC]) {
        if (s >= 0) {
            load_row(s, row);
        } else {
#pragma unroll
            for (int e = 0; e < VEC; e++)
                row[e] = p.input_state == nullptr
                             ? 0.f
                             : (float)reinterpret_cast<const T*>(p.input_state)[((int64_t)b * p.C + c0 + e) * (KS - 1) + (KS - 1) + s];
        }
    };
    auto emit = [&](int s, const float (&cur)[VEC], const float (&hist)[KS - 1][VEC]) {  // hist[j] = row s - (KS - 1) + j
        const float m = mb == nullptr ? 1.f : (float)mb[s];
        vec_t out;
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            float acc = bias[e] + wflat[e * KS + KS - 1] * cur[e];
#pragma unroll
            for (int j = 0; j < KS - 1; j++) acc += wflat[e * KS + j] * hist[j][e];
            if (SILU) acc = acc * __builtin_amdgcn_rcpf(1.f + __expf(-acc));  // x * sigmoid(x)
            out[e] = (T)(acc * m);
        }
        *reinterpret_cast<vec_t*>(yb + (int64_t)s * p.y_stride_s) = out;
    };

    // Token blocks are walked in alternating directions: an even block from its last token down, an odd one
    // from its first token up.  The kernel_size - 1 rows two neighbouring blocks have in common are then read
    // by both at the same moment - at the start of both walks or at the end of both - and come out of the
    // cache; walked the same way, the second reader comes a whole walk later and fetches them from memory
    // again (measured: 19 % more bytes fetched than the input holds, 5 % this way; the kernel time did not
    // change, it streams at the rate of a plain copy either way).
    const bool downward = ((s_begin / CONV_TOKENS) & 1) == 0;
    float hist[KS - 1][VEC];
    if (!downward) {
#pragma unroll
        for (int j = 0; j < KS - 1; j++) load_any(s_begin - (KS - 1) + j, hist[j]);
#pragma unroll 8
        for (int s = s_begin; s < s_end; s++) {
            float cur[VEC];
            load_row(s, cur);
            emit(s, cur, hist);
#pragma unroll
            for (int e = 0; e < VEC; e++) {
#pragma unroll
                for (int j = 0; j + 1 < KS - 1; j++) hist[j][e] = hist[j + 1][e];
                hist[KS - 2][e] = cur[e];
            }
        }
        if (p.final_state != nullptr && s_end == p.S) {
            T* fs = reinterpret_cast<T*>(p.final_state) + ((int64_t)b * p.C + c0) * (KS - 1);
#pragma unroll
            for (int e = 0; e < VEC; e++)
#pragma unroll
                for (int j = 0; j < KS - 1; j++) fs[e * (KS - 1) + j] = (T)hist[j][e];
        }
    } else {
        // cur = row s, hist[j] = row s - (KS - 1) + j; stepping down shifts the window the other way
        float cur[VEC];
        load_row(s_end - 1, cur);
#pragma unroll
        for (int j = 0; j < KS - 1; j++) load_any(s_end - 1 - (KS - 1) + j, hist[j]);
        if (p.final_state != nullptr && s_end == p.S) {  // the last kernel_size - 1 inputs: hist[1..], cur
            T* fs = reinterpret_cast<T*>(p.final_state) + ((int64_t)b * p.C + c0) * (KS - 1);
#pragma unroll
            for (int e = 0; e < VEC; e++) {
#pragma unroll
                for (int j = 0; j + 1 < KS - 1; j++) fs[e * (KS - 1) + j] = (T)hist[j + 1][e];
                fs[e * (KS - 1) + KS - 2] = (T)cur[e];
            }
        }
#pragma unroll 8
        for (int s = s_end - 1; s >= s_begin; s--) {
            emit(s, cur, hist);
            float next[VEC] = {};  // row s - KS, the new oldest row of the window around s - 1
            if (s > s_begin) load_any(s - KS, next);
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                cur[e] = hist[KS - 2][e];
#pragma unroll
                for (int j = KS - 2; j > 0; j--) hist[j][e] = hist[j - 1][e];
                hist[0][e] = next[e];
            }
        }
    }
}

template <typename T, typename WT, int KS>
static void launch_conv_ks(const ConvParams& p, bool silu, dim3 grid, hipStream_t stream) {
    if (silu) hipLaunchKernelGGL((causal_conv1d_kernel<T, WT, KS, true>), grid, dim3(CONV_THREADS), 0, stream, p);
    else hipLaunchKernelGGL((causal_conv1d_kernel<T, WT, KS, false>), grid, dim3(CONV_THREADS), 0, stream, p);
}

template <typename T, typename WT>
static int launch_conv(const ConvParams& p, int kernel_size, bool silu, hipStream_t stream) {
    const int vecs = p.C / ConvVec<T>::N;
    constexpr int SPAN = (CONV_THREADS / WAVE) * CONV_TOKENS;  // tokens per workgroup
    const dim3 grid((vecs + WAVE - 1) / WAVE, (p.S + SPAN - 1) / SPAN, p.B);
    if (kernel_size == 2) launch_conv_ks<T, WT, 2>(p, silu, grid, stream);
    else if (kernel_size == 3) launch_conv_ks<T, WT, 3>(p, silu, grid, stream);
    else launch_conv_ks<T, WT, 4>(p, silu, grid, stream);
    return (int)hipGetLastError();
}

}  // namespace gdn

namespace {
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) % 16) == 0; }
}  // namespace

extern "C" int gdn_causal_conv1d_fwd(const gdn_conv_args* a, void* stream) {
    if (a == nullptr || a->x == nullptr || a->y == nullptr || a->weight == nullptr) return GDN_ERR_NULL;
    if (a->B <= 0 || a->S <= 0 || a->C <= 0) return GDN_ERR_SHAPE;
    if (a->kernel_size < 2 || a->kernel_size > 4) return GDN_ERR_UNSUPPORTED;
    if (a->dtype != GDN_BF16 && a->dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    if (a->w_dtype != GDN_BF16 && a->w_dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    if (a->dtype == GDN_F32 && a->w_dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;  // weights as wide as the data
    if (a->activation != GDN_ACT_NONE && a->activation != GDN_ACT_SILU) return GDN_ERR_UNSUPPORTED;
    if (a->B > 65535 || a->S / (gdn::CONV_TOKENS * (gdn::CONV_THREADS / gdn::WAVE)) >= 65535) return GDN_ERR_UNSUPPORTED;
    const int64_t vec = (a->dtype == GDN_BF16) ? 8 : 4;
    if (a->C % vec != 0) return GDN_ERR_UNSUPPORTED;
    const int64_t strides[] = {a->x_stride_b, a->x_stride_s, a->y_stride_b, a->y_stride_s};
    for (int64_t s : strides)
        if (s < 0 || s % vec != 0) return GDN_ERR_ALIGN;
    if (a->x_stride_s < a->C || a->y_stride_s < a->C) return GDN_ERR_SHAPE;
    if (!aligned16(a->x) || !aligned16(a->y) || !aligned16(a->weight) || (a->bias && !aligned16(a->bias))) return GDN_ERR_ALIGN;
    if (a->x == a->y) return GDN_ERR_SHAPE;  // neighbouring token blocks re-read rows of x

    gdn::ConvParams p;
    p.x = a->x, p.weight = a->weight, p.bias = a->bias, p.input_state = a->input_state, p.mask = a->mask;
    p.y = a->y, p.final_state = a->final_state;
    p.x_stride_b = a->x_stride_b, p.x_stride_s = a->x_stride_s;
    p.y_stride_b = a->y_stride_b, p.y_stride_s = a->y_stride_s;
    p.B = a->B, p.S = a->S, p.C = a->C;
    const bool silu = a->activation == GDN_ACT_SILU;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (a->dtype == GDN_BF16 && a->w_dtype == GDN_BF16) return gdn::launch_conv<gdn::bf16_t, gdn::bf16_t>(p, a->kernel_size, silu, st);
    if (a->dtype == GDN_BF16) return gdn::launch_conv<gdn::bf16_t, float>(p, a->kernel_size, silu, st);
    return gdn::launch_conv<float, float>(p, a->kernel_size, silu, st);
}
