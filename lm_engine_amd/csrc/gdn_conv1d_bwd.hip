// Backward of the depthwise causal convolution (kernel size 2..4, bias, optional SiLU, optional padding mask,
// optional carried-in state): what autograd computes through DepthwiseCausalConvolution.forward,
// lm_engine/modeling_utils/depthwise_causal_convolution.py:103-241, when the layer trains.
//
// Forward, per channel: xx = [state or zeros (KS - 1 rows) | x * mask], z[s] = bias + sum_j w[j] xx[s + j],
// y[s] = act(z[s]) * mask[s].  Backward with dz[s] = dy[s] mask[s] act'(z[s]):
//     dxx[u]  = sum_j w[j] dz[u - j]           dx[t] = mask[t] dxx[t + KS - 1]      dstate[i] = dxx[i]
//     dw[j]   = sum_{b, s} dz[s] xx[s + j]     dbias = sum_{b, s} dz[s]
// One pass: a thread owns 2 consecutive channels and walks a block of tokens upward, recomputing z from a
// sliding window of xx (nothing was saved by the forward), keeping KS partial sums of dxx in flight, and
// accumulating dw and dbias for its block in registers; the KS - 1 rows of dz past the block's end are recomputed
// for dx only.  The per-block partial sums of dw and dbias go to a [blocks][C] array each that the caller adds up.
#include <hip/hip_runtime.h>

#include "gdn_common.h"
#include "gdn_launch.h"

namespace gdn {

namespace {

constexpr int CB_THREADS = 256;
// Channels per thread.  The kernel is bound by its arithmetic (about 35 vector instructions per token and channel against
// 6 bytes), so narrow accesses that put more waves on a CU beat 16-byte ones: at B = 4, S = 4096, C = 6144 bf16, kernel plus
// the two sums of the partial results, 8 channels 189 us, 4 channels 173 us, 2 channels (8 rows in flight, 256 tokens
// per block) 163 us.
constexpr int CB_VEC = 2;

struct ConvBwdParams {
    const void* x;  // x, dy, input_state, mask, dx, dstate: bf16 or fp32 (the kernel's T)
    const void* dy;
    const void* weight;
    const void* bias;
    const void* input_state;
    const void* mask;
    void* dx;
    void* dstate;
    float* dw_part;  // [B * blocks per row][C][KS]
    float* db_part;  // [B * blocks per row][C]
    int64_t x_stride_b, x_stride_s, dy_stride_b, dy_stride_s;
    int B, S, C;
    int w_is_bf16;
    int tokens_per_block;  // tokens per block of the walk
};

__device__ __forceinline__ float load_w(const void* w, int is_bf16, int64_t i) {
    return is_bf16 ? (float)reinterpret_cast<const bf16_t*>(w)[i] : reinterpret_cast<const float*>(w)[i];
}

// T: element type of the activations; VEC consecutive channels per thread, one vector access per row
template <typename T, int KS, bool SILU, int VEC, bool MASK>
__global__ __launch_bounds__(CB_THREADS) void causal_conv1d_bwd_kernel(const ConvBwdParams p) {
    typedef T vec_t __attribute__((ext_vector_type(VEC)));
    const int c0 = (blockIdx.x * CB_THREADS + threadIdx.x) * VEC;
    if (c0 >= p.C) return;
    const int blocks_per_row = (p.S + p.tokens_per_block - 1) / p.tokens_per_block;
    const int b = blockIdx.y / blocks_per_row, blk = blockIdx.y % blocks_per_row;
    const int s_begin = blk * p.tokens_per_block;
    const int s_own = min(s_begin + p.tokens_per_block, p.S);      // dz of [s_begin, s_own) belongs to this block
    const int s_end = min(s_own + KS - 1, p.S);           // dz up to here feeds dx of this block

    const T* xb = static_cast<const T*>(p.x) + (int64_t)b * p.x_stride_b + c0;
    const T* dyb = static_cast<const T*>(p.dy) + (int64_t)b * p.dy_stride_b + c0;
    const T* mb = MASK ? static_cast<const T*>(p.mask) + (int64_t)b * p.S : nullptr;  // MASK is false when there is none
    T* dxb = static_cast<T*>(p.dx) + ((int64_t)b * p.S) * p.C + c0;
    const T* const state_in = static_cast<const T*>(p.input_state);
    T* const state_out = static_cast<T*>(p.dstate);

    float w[VEC][KS], bias[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) {
#pragma unroll
        for (int j = 0; j < KS; j++) w[e][j] = load_w(p.weight, p.w_is_bf16, (int64_t)(c0 + e) * KS + j);
        bias[e] = p.bias == nullptr ? 0.f : load_w(p.bias, p.w_is_bf16, c0 + e);
    }

    // row s of xx in x's index (s < 0: carried state or zeros)
    auto load_xx = [&](int s, float (&row)[VEC]) {
        if (s >= 0) {
            const vec_t v = *reinterpret_cast<const vec_t*>(xb + (int64_t)s * p.x_stride_s);
            const float m = MASK ? (float)mb[s] : 1.f;
#pragma unroll
            for (int e = 0; e < VEC; e++) row[e] = (float)v[e] * m;
        } else {
#pragma unroll
            for (int e = 0; e < VEC; e++)
                row[e] = state_in == nullptr ? 0.f : (float)state_in[((int64_t)b * p.C + c0 + e) * (KS - 1) + (KS - 1) + s];
        }
    };

    float win[KS][VEC];   // win[j] = xx row (s - (KS - 1) + j) for the current s
    float pend[KS][VEC];  // pend[j] = partial dxx of x index (s - (KS - 1) + j)
    float dw[VEC][KS], db[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        db[e] = 0.f;
#pragma unroll
        for (int j = 0; j < KS; j++) dw[e][j] = 0.f, pend[j][e] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < KS - 1; j++) load_xx(s_begin - (KS - 1) + j, win[j + 1]);  // shifted into place by the first step

    // The walk goes in steps of UNROLL tokens whose rows of x and dy are all requested before the first is used: a
    // thread then has 2 UNROLL loads in flight instead of two, which is what a streaming kernel with this few waves
    // per CU needs to keep the memory system busy.  (Rows past s_end are read again from row s_end - 1 and not used.)
    constexpr int UNROLL = 8;
    for (int s0 = s_begin; s0 < s_end; s0 += UNROLL) {
        vec_t xr[UNROLL], gr[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const int su = min(s0 + u, s_end - 1);
            xr[u] = *reinterpret_cast<const vec_t*>(xb + (int64_t)su * p.x_stride_s);
            gr[u] = *reinterpret_cast<const vec_t*>(dyb + (int64_t)su * p.dy_stride_s);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const int s = s0 + u;
            if (s >= s_end) break;
            // slide: win[j] <- win[j + 1], pend likewise (pend[0] of the last step was emitted below)
#pragma unroll
            for (int e = 0; e < VEC; e++) {
#pragma unroll
                for (int j = 0; j + 1 < KS; j++) win[j][e] = win[j + 1][e], pend[j][e] = pend[j + 1][e];
                pend[KS - 1][e] = 0.f;
            }
            const float m = MASK ? (float)mb[s] : 1.f;
#pragma unroll
            for (int e = 0; e < VEC; e++) win[KS - 1][e] = (float)xr[u][e] * m;
            const vec_t g = gr[u];
            const bool own = s < s_own;
#pragma unroll
            for (int e = 0; e < VEC; e++) {
                float z = bias[e];
#pragma unroll
                for (int j = 0; j < KS; j++) z += w[e][j] * win[j][e];
                float dz = (float)g[e] * m;
                if (SILU) {
                    const float sg = __builtin_amdgcn_rcpf(1.f + __expf(-z));
                    dz *= sg * (1.f + z * (1.f - sg));
                }
#pragma unroll
                for (int j = 0; j < KS; j++) pend[j][e] += w[e][j] * dz;  // x index s - (KS - 1) + j
                if (own) {
                    db[e] += dz;
#pragma unroll
                    for (int j = 0; j < KS; j++) dw[e][j] += dz * win[j][e];
                }
            }
            // x index t = s - (KS - 1) is complete now
            const int t = s - (KS - 1);
            if (t >= s_begin) {
                const float mt = MASK ? (float)mb[t] : 1.f;
                vec_t out;
#pragma unroll
                for (int e = 0; e < VEC; e++) out[e] = (T)(pend[0][e] * mt);
                __builtin_nontemporal_store(out, reinterpret_cast<vec_t*>(dxb + (int64_t)t * p.C));  // (nobody reads dx back soon)
            } else if (t < 0 && state_out != nullptr) {  // only in the first block of a row
#pragma unroll
                for (int e = 0; e < VEC; e++) state_out[((int64_t)b * p.C + c0 + e) * (KS - 1) + (KS - 1) + t] = (T)pend[0][e];
            }
        }
    }
    // the rows still in flight: x indices s_end - (KS - 1) + 1 .. s_end - 1 (complete only at the end of the sequence;
    // inside it they belong to the next block, which recomputes them)
    if (s_end == p.S) {
#pragma unroll
        for (int j = 1; j < KS; j++) {
            const int t = s_end - 1 - (KS - 1) + j;
            if (t >= s_begin && t < s_own) {
                const float mt = MASK ? (float)mb[t] : 1.f;
                vec_t out;
#pragma unroll
                for (int e = 0; e < VEC; e++) out[e] = (T)(pend[j][e] * mt);
                __builtin_nontemporal_store(out, reinterpret_cast<vec_t*>(dxb + (int64_t)t * p.C));  // (nobody reads dx back soon)
            } else if (t < 0 && t >= -(KS - 1) && s_begin == 0 && state_out != nullptr) {
#pragma unroll
                for (int e = 0; e < VEC; e++) state_out[((int64_t)b * p.C + c0 + e) * (KS - 1) + (KS - 1) + t] = (T)pend[j][e];
            }
        }
    }
    const int64_t part = (int64_t)blockIdx.y * p.C + c0;
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        p.db_part[part + e] = db[e];
#pragma unroll
        for (int j = 0; j < KS; j++) p.dw_part[(part + e) * KS + j] = dw[e][j];
    }
}

template <typename T, int KS>
int launch_ks(const ConvBwdParams& p, bool silu, hipStream_t stream) {
    constexpr int VEC = CB_VEC;
    const int blocks_per_row = (p.S + p.tokens_per_block - 1) / p.tokens_per_block;
    const dim3 grid((unsigned)((p.C / VEC + CB_THREADS - 1) / CB_THREADS), (unsigned)(p.B * blocks_per_row));
    const bool mask = p.mask != nullptr;
    if (silu && mask) hipLaunchKernelGGL((causal_conv1d_bwd_kernel<T, KS, true, VEC, true>), grid, dim3(CB_THREADS), 0, stream, p);
    else if (silu) hipLaunchKernelGGL((causal_conv1d_bwd_kernel<T, KS, true, VEC, false>), grid, dim3(CB_THREADS), 0, stream, p);
    else if (mask) hipLaunchKernelGGL((causal_conv1d_bwd_kernel<T, KS, false, VEC, true>), grid, dim3(CB_THREADS), 0, stream, p);
    else hipLaunchKernelGGL((causal_conv1d_bwd_kernel<T, KS, false, VEC, false>), grid, dim3(CB_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}

template <typename T>
int launch_t(const ConvBwdParams& p, int kernel_size, bool silu, hipStream_t stream) {
    switch (kernel_size) {
        case 2: return launch_ks<T, 2>(p, silu, stream);
        case 3: return launch_ks<T, 3>(p, silu, stream);
        case 4: return launch_ks<T, 4>(p, silu, stream);
        default: return GDN_ERR_UNSUPPORTED;
    }
}

}  // namespace

int launch_conv_bwd(const gdn_conv_bwd_args& a, hipStream_t stream) {
    ConvBwdParams p;
    p.x = a.x, p.dy = a.dy;
    p.weight = a.weight, p.bias = a.bias;
    p.input_state = a.input_state, p.mask = a.mask;
    p.dx = a.dx, p.dstate = a.dstate;
    p.dw_part = a.dweight_partial, p.db_part = a.dbias_partial;
    p.x_stride_b = a.x_stride_b, p.x_stride_s = a.x_stride_s, p.dy_stride_b = a.dy_stride_b, p.dy_stride_s = a.dy_stride_s;
    p.B = a.B, p.S = a.S, p.C = a.C;
    p.w_is_bf16 = a.w_dtype == GDN_BF16 ? 1 : 0;
    p.tokens_per_block = a.tokens_per_block;
    const bool silu = a.activation == GDN_ACT_SILU;
    return a.dtype == GDN_BF16 ? launch_t<bf16_t>(p, a.kernel_size, silu, stream) : launch_t<float>(p, a.kernel_size, silu, stream);
}

}  // namespace gdn
