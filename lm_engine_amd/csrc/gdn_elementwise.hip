// The two elementwise / row-wise steps of the layer on either side of the operator, each as one
// pass over HBM:
//
//   gates     g = -exp(A_log) * softplus(a + dt_bias)  (fp32),  beta = scale * sigmoid(b)
//   epilogue  y = rmsnorm(o * silu(gate)) * weight  over the V columns of each (token, head)
//
// Both are HBM-bound.  Algorithmic bytes: gates 2 + 2 in, 4 + 2 out per (token, head) with bf16
// activations; epilogue 3 elements (o and gate in, y out) per (token, head, column).

#include "gdn_common.h"

namespace gdn {

struct GateParams {
    const void* a;
    const void* b;
    const float* A_log;
    const float* dt_bias;
    float* g;
    void* beta;
    int64_t a_stride, b_stride;
    int64_t tokens;
    int H;
    float beta_scale;
};

// F.softplus with its default threshold: x for x > 20, log1p(exp(x)) otherwise
__device__ __forceinline__ float softplus(float x) { return x > 20.f ? x : log1pf(__expf(x)); }

template <typename T>
__global__ __launch_bounds__(256) void gates_kernel(const GateParams p) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= p.tokens * p.H) return;
    const int64_t t = idx / p.H;
    const int h = (int)(idx % p.H);
    const float a = (float)reinterpret_cast<const T*>(p.a)[t * p.a_stride + h];
    const float b = (float)reinterpret_cast<const T*>(p.b)[t * p.b_stride + h];
    p.g[idx] = -expf(p.A_log[h]) * softplus(a + p.dt_bias[h]);
    // sigmoid in fp32, rounded to the activation dtype, then scaled in that dtype like `b.sigmoid() * 2`
    const T s = (T)(1.f / (1.f + expf(-b)));
    reinterpret_cast<T*>(p.beta)[idx] = (T)((float)s * p.beta_scale);
}

// Backward of the gates: with z = a + dt_bias, rate = -exp(A_log), s = sigmoid(b)
//     da = d_dt_bias terms = dg rate sigmoid(z)       dA_log = sum dg rate softplus(z)       db = dbeta scale s (1 - s)
// A thread walks the flat (token, head) index with a stride that is a multiple of H, so it stays on one head and keeps
// that head's two sums in registers; a workgroup leaves them, added up per head in a fixed order, in row blockIdx.x of
// the two partial arrays, which the caller adds up over the rows.
struct GateBwdParams {
    const void* a;
    const void* b;
    const float* A_log;
    const float* dt_bias;
    const float* dg;
    const void* dbeta;
    void* da;
    void* db;
    float* dA_part;   // [gridDim.x][H]
    float* ddt_part;  // [gridDim.x][H]
    int64_t a_stride, b_stride;
    int64_t tokens;
    int H;
    float beta_scale;
};

template <typename T>
__global__ __launch_bounds__(256) void gates_bwd_kernel(const GateBwdParams p) {
    __shared__ float s_A[256], s_dt[256];
    const int64_t n = p.tokens * p.H;
    const int64_t stride = ((int64_t)gridDim.x * 256 + p.H - 1) / p.H * p.H;  // a multiple of H
    const int64_t first = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int h = (int)(first % p.H);
    const float rate = -expf(p.A_log[h]), bias = p.dt_bias[h];
    float acc_A = 0.f, acc_dt = 0.f;
    for (int64_t idx = first; idx < n; idx += stride) {
        const int64_t t = idx / p.H;
        const float z = (float)reinterpret_cast<const T*>(p.a)[t * p.a_stride + h] + bias;
        const float b = (float)reinterpret_cast<const T*>(p.b)[t * p.b_stride + h];
        const float dg = p.dg[idx];
        const float dz = dg * rate * (1.f / (1.f + expf(-z)));
        const float s = 1.f / (1.f + expf(-b));
        reinterpret_cast<T*>(p.da)[idx] = (T)dz;
        reinterpret_cast<T*>(p.db)[idx] = (T)((float)reinterpret_cast<const T*>(p.dbeta)[idx] * p.beta_scale * s * (1.f - s));
        acc_A += dg * rate * softplus(z);
        acc_dt += dz;
    }
    s_A[threadIdx.x] = acc_A, s_dt[threadIdx.x] = acc_dt;
    __syncthreads();
    for (int hh = threadIdx.x; hh < p.H; hh += 256) {  // thread i of this workgroup sits on head (blockIdx.x * 256 + i) % H
        float sum_A = 0.f, sum_dt = 0.f;
        int i = (int)((hh - (int64_t)blockIdx.x * 256 % p.H + p.H) % p.H);
        for (; i < 256; i += p.H) sum_A += s_A[i], sum_dt += s_dt[i];
        p.dA_part[(int64_t)blockIdx.x * p.H + hh] = sum_A;
        p.ddt_part[(int64_t)blockIdx.x * p.H + hh] = sum_dt;
    }
}

// 8 consecutive elements <-> fp32, with 16-byte accesses
__device__ __forceinline__ void load8(const bf16_t* p, float (&x)[8]) {
    const bf16x8 v = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
    for (int e = 0; e < 8; e++) x[e] = (float)v[e];
}
__device__ __forceinline__ void load8(const float* p, float (&x)[8]) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
    for (int e = 0; e < 4; e++) x[e] = a[e], x[4 + e] = b[e];
}
__device__ __forceinline__ void store8(bf16_t* p, const float (&x)[8]) {
    bf16x8 v;
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = (bf16_t)x[e];
    *reinterpret_cast<bf16x8*>(p) = v;
}
__device__ __forceinline__ void store8(float* p, const float (&x)[8]) {
    *reinterpret_cast<f32x4*>(p) = f32x4{x[0], x[1], x[2], x[3]};
    *reinterpret_cast<f32x4*>(p + 4) = f32x4{x[4], x[5], x[6], x[7]};
}

// the same with non-temporal stores (streams that nobody reads again soon)
__device__ __forceinline__ void store8_stream(bf16_t* p, const float (&x)[8]) {
    bf16x8 v;
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = (bf16_t)x[e];
    __builtin_nontemporal_store(v, reinterpret_cast<bf16x8*>(p));
}
__device__ __forceinline__ void store8_stream(float* p, const float (&x)[8]) {
    __builtin_nontemporal_store(f32x4{x[0], x[1], x[2], x[3]}, reinterpret_cast<f32x4*>(p));
    __builtin_nontemporal_store(f32x4{x[4], x[5], x[6], x[7]}, reinterpret_cast<f32x4*>(p + 4));
}

struct NormParams {
    const void* o;
    const void* gate;
    const void* weight;
    void* y;
    int64_t o_stride_t, gate_stride_t, y_stride_t;
    int64_t rows;  // tokens * H
    int H, V;
    float eps;
};

// LPR lanes per row, 8 consecutive columns per lane (16-byte accesses for bf16, 2 x 16 for fp32)
template <typename T, typename WT, int LPR>
__global__ __launch_bounds__(256) void gated_rmsnorm_kernel(const NormParams p) {
    constexpr int ROWS_PER_BLOCK = 256 / LPR;
    const int sub = threadIdx.x % LPR;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_BLOCK + threadIdx.x / LPR;
    const bool live = row < p.rows && sub * 8 < p.V;
    const int64_t t = live ? row / p.H : 0;
    const int h = live ? (int)(row % p.H) : 0;
    const int c = sub * 8;

    float x[8];
#pragma unroll
    for (int e = 0; e < 8; e++) x[e] = 0.f;
    if (live) {
        load8(reinterpret_cast<const T*>(p.o) + t * p.o_stride_t + (int64_t)h * p.V + c, x);
        if (p.gate != nullptr) {
            float g[8];
            load8(reinterpret_cast<const T*>(p.gate) + t * p.gate_stride_t + (int64_t)h * p.V + c, g);
#pragma unroll
            for (int e = 0; e < 8; e++) x[e] *= g[e] * __builtin_amdgcn_rcpf(1.f + __expf(-g[e]));
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) ss += x[e] * x[e];
#pragma unroll
    for (int off = 1; off < LPR; off <<= 1) ss += __shfl_xor(ss, off, WAVE);
    if (!live) return;
    const float r = rsqrtf(ss / (float)p.V + p.eps);
    float w[8];
#pragma unroll
    for (int e = 0; e < 8; e++) w[e] = 1.f;
    if (p.weight != nullptr) load8(reinterpret_cast<const WT*>(p.weight) + c, w);
#pragma unroll
    for (int e = 0; e < 8; e++) x[e] = x[e] * r * w[e];
    store8(reinterpret_cast<T*>(p.y) + t * p.y_stride_t + (int64_t)h * p.V + c, x);
}

template <typename T, typename WT>
static int launch_norm(const NormParams& p, hipStream_t stream) {
    int lpr = 8;
    while (lpr * 8 < p.V) lpr *= 2;
    const int64_t rows_per_block = 256 / lpr;
    const dim3 grid((unsigned)((p.rows + rows_per_block - 1) / rows_per_block));
    if (lpr == 8) hipLaunchKernelGGL((gated_rmsnorm_kernel<T, WT, 8>), grid, dim3(256), 0, stream, p);
    else if (lpr == 16) hipLaunchKernelGGL((gated_rmsnorm_kernel<T, WT, 16>), grid, dim3(256), 0, stream, p);
    else if (lpr == 32) hipLaunchKernelGGL((gated_rmsnorm_kernel<T, WT, 32>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((gated_rmsnorm_kernel<T, WT, 64>), grid, dim3(256), 0, stream, p);
    return (int)hipGetLastError();
}

// Backward of gated_rmsnorm_kernel: with x = o silu(g), r = (mean(x^2) + eps)^-1/2, y = x r w,
//     dx = r (dy w) - (r^3 / V) x <dy w, x>     do = dx silu(g)     dg = dx o silu'(g)     dw = sum_rows dy x r
// Same lane mapping; a workgroup walks over row groups with a stride of the grid and leaves its partial sum of
// dw in dw_part[blockIdx.x][V] (fp32), which the caller adds up.
struct NormBwdParams {
    const void* o;
    const void* gate;
    const void* weight;
    const void* dy;
    void* d_o;
    void* d_gate;
    float* dw_part;
    int64_t o_stride_t, gate_stride_t;
    int64_t rows;
    int H, V;
    float eps;
};

template <typename T, typename WT, int LPR>
__global__ __launch_bounds__(256) void gated_rmsnorm_bwd_kernel(const NormBwdParams p) {
    constexpr int ROWS_PER_BLOCK = 256 / LPR;
    __shared__ float s_dw[ROWS_PER_BLOCK][LPR * 8];
    const int sub = threadIdx.x % LPR, slot = threadIdx.x / LPR;
    const int c = sub * 8;
    const bool col_live = c < p.V;
    float w[8], dw[8];
#pragma unroll
    for (int e = 0; e < 8; e++) w[e] = 1.f, dw[e] = 0.f;
    if (col_live && p.weight != nullptr) load8(reinterpret_cast<const WT*>(p.weight) + c, w);
    const int64_t groups = (p.rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
    for (int64_t grp = blockIdx.x; grp < groups; grp += gridDim.x) {
        const int64_t row = grp * ROWS_PER_BLOCK + slot;
        const bool live = row < p.rows && col_live;
        const int64_t t = live ? row / p.H : 0;
        const int h = live ? (int)(row % p.H) : 0;
        float o[8], g[8], dy[8], x[8], sg[8];
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] = 0.f, g[e] = 0.f, dy[e] = 0.f, sg[e] = 1.f;
        if (live) {
            load8(reinterpret_cast<const T*>(p.o) + t * p.o_stride_t + (int64_t)h * p.V + c, o);
            load8(reinterpret_cast<const T*>(p.dy) + row * p.V + c, dy);
            if (p.gate != nullptr) load8(reinterpret_cast<const T*>(p.gate) + t * p.gate_stride_t + (int64_t)h * p.V + c, g);
        }
        float ss = 0.f, dot = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            if (p.gate != nullptr) sg[e] = __builtin_amdgcn_rcpf(1.f + __expf(-g[e]));
            x[e] = p.gate != nullptr ? o[e] * g[e] * sg[e] : o[e];
            ss += x[e] * x[e];
            dot += dy[e] * w[e] * x[e];
        }
#pragma unroll
        for (int off = 1; off < LPR; off <<= 1) ss += __shfl_xor(ss, off, WAVE), dot += __shfl_xor(dot, off, WAVE);
        if (live) {
            const float r = rsqrtf(ss / (float)p.V + p.eps);
            const float k = r * r * r * dot / (float)p.V;
            float d_o[8], d_g[8];
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float dx = r * dy[e] * w[e] - k * x[e];
                dw[e] += dy[e] * x[e] * r;
                if (p.gate != nullptr) {
                    d_o[e] = dx * g[e] * sg[e];
                    d_g[e] = dx * o[e] * sg[e] * (1.f + g[e] * (1.f - sg[e]));
                } else {
                    d_o[e] = dx;
                }
            }
            // non-temporal: nobody reads the gradients back soon, and they would push o, gate and dy out of the cache
            // (76 -> 68 us at 4 x 4096 x 16 x 128; non-temporal loads on top of that lose it again)
            store8_stream(reinterpret_cast<T*>(p.d_o) + row * p.V + c, d_o);
            if (p.gate != nullptr) store8_stream(reinterpret_cast<T*>(p.d_gate) + row * p.V + c, d_g);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) s_dw[slot][c + e] = dw[e];
    __syncthreads();
    if (slot == 0 && col_live) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float acc = 0.f;
            for (int q = 0; q < ROWS_PER_BLOCK; q++) acc += s_dw[q][c + e];
            p.dw_part[(int64_t)blockIdx.x * p.V + c + e] = acc;
        }
    }
}

template <typename T, typename WT>
static int launch_norm_bwd(const NormBwdParams& p, int blocks, hipStream_t stream) {
    int lpr = 8;
    while (lpr * 8 < p.V) lpr *= 2;
    const dim3 grid((unsigned)blocks);
    if (lpr == 8) hipLaunchKernelGGL((gated_rmsnorm_bwd_kernel<T, WT, 8>), grid, dim3(256), 0, stream, p);
    else if (lpr == 16) hipLaunchKernelGGL((gated_rmsnorm_bwd_kernel<T, WT, 16>), grid, dim3(256), 0, stream, p);
    else if (lpr == 32) hipLaunchKernelGGL((gated_rmsnorm_bwd_kernel<T, WT, 32>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((gated_rmsnorm_bwd_kernel<T, WT, 64>), grid, dim3(256), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace gdn

namespace {
inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
}  // namespace

extern "C" int gdn_gates_fwd(const gdn_gate_args* a, void* stream) {
    if (a == nullptr || !a->a || !a->b || !a->A_log || !a->dt_bias || !a->g || !a->beta) return GDN_ERR_NULL;
    if (a->tokens <= 0 || a->H <= 0) return GDN_ERR_SHAPE;
    if (a->a_stride < a->H || a->b_stride < a->H) return GDN_ERR_SHAPE;
    if (a->dtype != GDN_BF16 && a->dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    const int64_t blocks = (a->tokens * (int64_t)a->H + 255) / 256;
    if (blocks > 0x7fffffff) return GDN_ERR_UNSUPPORTED;
    gdn::GateParams p;
    p.a = a->a, p.b = a->b, p.A_log = a->A_log, p.dt_bias = a->dt_bias, p.g = a->g, p.beta = a->beta;
    p.a_stride = a->a_stride, p.b_stride = a->b_stride, p.tokens = a->tokens, p.H = a->H, p.beta_scale = a->beta_scale;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (a->dtype == GDN_BF16) hipLaunchKernelGGL((gdn::gates_kernel<gdn::bf16_t>), dim3((unsigned)blocks), dim3(256), 0, st, p);
    else hipLaunchKernelGGL((gdn::gates_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, st, p);
    return (int)hipGetLastError();
}

extern "C" int gdn_gates_bwd(const gdn_gate_bwd_args* a, void* stream) {
    if (a == nullptr || !a->a || !a->b || !a->A_log || !a->dt_bias || !a->dg || !a->dbeta || !a->da || !a->db || !a->dA_log_partial ||
        !a->ddt_bias_partial)
        return GDN_ERR_NULL;
    if (a->tokens <= 0 || a->H <= 0 || a->partial_blocks <= 0 || a->partial_blocks > 65535) return GDN_ERR_SHAPE;
    if (a->a_stride < a->H || a->b_stride < a->H) return GDN_ERR_SHAPE;
    if (a->dtype != GDN_BF16 && a->dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    gdn::GateBwdParams p;
    p.a = a->a, p.b = a->b, p.A_log = a->A_log, p.dt_bias = a->dt_bias, p.dg = a->dg, p.dbeta = a->dbeta;
    p.da = a->da, p.db = a->db, p.dA_part = a->dA_log_partial, p.ddt_part = a->ddt_bias_partial;
    p.a_stride = a->a_stride, p.b_stride = a->b_stride, p.tokens = a->tokens, p.H = a->H, p.beta_scale = a->beta_scale;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (a->dtype == GDN_BF16) hipLaunchKernelGGL((gdn::gates_bwd_kernel<gdn::bf16_t>), dim3((unsigned)a->partial_blocks), dim3(256), 0, st, p);
    else hipLaunchKernelGGL((gdn::gates_bwd_kernel<float>), dim3((unsigned)a->partial_blocks), dim3(256), 0, st, p);
    return (int)hipGetLastError();
}

extern "C" int gdn_gated_rmsnorm_fwd(const gdn_norm_args* a, void* stream) {
    if (a == nullptr || !a->o || !a->y) return GDN_ERR_NULL;
    if (a->tokens <= 0 || a->H <= 0 || a->V <= 0) return GDN_ERR_SHAPE;
    if (a->V % 8 != 0 || a->V > 512) return GDN_ERR_UNSUPPORTED;
    if (a->dtype != GDN_BF16 && a->dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    if (a->weight && a->w_dtype != GDN_BF16 && a->w_dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    const int64_t row_elems = (int64_t)a->H * a->V;
    if (a->o_stride_t < row_elems || a->y_stride_t < row_elems || (a->gate && a->gate_stride_t < row_elems)) return GDN_ERR_SHAPE;
    const size_t esz = a->dtype == GDN_BF16 ? 2 : 4;
    if (!aligned_to(a->o, 16) || !aligned_to(a->y, 16) || (a->gate && !aligned_to(a->gate, 16)) || (a->weight && !aligned_to(a->weight, 16))) return GDN_ERR_ALIGN;
    if ((a->o_stride_t * esz) % 16 || (a->y_stride_t * esz) % 16 || (a->gate && (a->gate_stride_t * esz) % 16)) return GDN_ERR_ALIGN;
    const int64_t rows = a->tokens * (int64_t)a->H;
    if (rows / 4 > 0x7fffffff) return GDN_ERR_UNSUPPORTED;
    gdn::NormParams p;
    p.o = a->o, p.gate = a->gate, p.weight = a->weight, p.y = a->y;
    p.o_stride_t = a->o_stride_t, p.gate_stride_t = a->gate_stride_t, p.y_stride_t = a->y_stride_t;
    p.rows = rows, p.H = a->H, p.V = a->V, p.eps = a->eps;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool wf32 = a->weight == nullptr || a->w_dtype == GDN_F32;
    if (a->dtype == GDN_BF16) return wf32 ? gdn::launch_norm<gdn::bf16_t, float>(p, st) : gdn::launch_norm<gdn::bf16_t, gdn::bf16_t>(p, st);
    return wf32 ? gdn::launch_norm<float, float>(p, st) : gdn::launch_norm<float, gdn::bf16_t>(p, st);
}

extern "C" int gdn_gated_rmsnorm_bwd(const gdn_norm_bwd_args* a, void* stream) {
    if (a == nullptr || !a->o || !a->dy || !a->d_o || !a->dweight_partial) return GDN_ERR_NULL;
    if ((a->gate == nullptr) != (a->d_gate == nullptr)) return GDN_ERR_NULL;
    if (a->tokens <= 0 || a->H <= 0 || a->V <= 0 || a->partial_blocks <= 0) return GDN_ERR_SHAPE;
    if (a->V % 8 != 0 || a->V > 512) return GDN_ERR_UNSUPPORTED;
    if (a->dtype != GDN_BF16 && a->dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    if (a->weight && a->w_dtype != GDN_BF16 && a->w_dtype != GDN_F32) return GDN_ERR_UNSUPPORTED;
    const int64_t row_elems = (int64_t)a->H * a->V;
    if (a->o_stride_t < row_elems || (a->gate && a->gate_stride_t < row_elems)) return GDN_ERR_SHAPE;
    const size_t esz = a->dtype == GDN_BF16 ? 2 : 4;
    const void* ptrs[] = {a->o, a->dy, a->d_o, a->gate, a->d_gate, a->weight};
    for (const void* x : ptrs)
        if (x != nullptr && !aligned_to(x, 16)) return GDN_ERR_ALIGN;
    if ((a->o_stride_t * esz) % 16 || (a->gate && (a->gate_stride_t * esz) % 16)) return GDN_ERR_ALIGN;
    gdn::NormBwdParams p;
    p.o = a->o, p.gate = a->gate, p.weight = a->weight, p.dy = a->dy, p.d_o = a->d_o, p.d_gate = a->d_gate;
    p.dw_part = a->dweight_partial;
    p.o_stride_t = a->o_stride_t, p.gate_stride_t = a->gate_stride_t;
    p.rows = a->tokens * (int64_t)a->H, p.H = a->H, p.V = a->V, p.eps = a->eps;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool wf32 = a->weight == nullptr || a->w_dtype == GDN_F32;
    if (a->dtype == GDN_BF16)
        return wf32 ? gdn::launch_norm_bwd<gdn::bf16_t, float>(p, a->partial_blocks, st)
                    : gdn::launch_norm_bwd<gdn::bf16_t, gdn::bf16_t>(p, a->partial_blocks, st);
    return wf32 ? gdn::launch_norm_bwd<float, float>(p, a->partial_blocks, st)
                : gdn::launch_norm_bwd<float, gdn::bf16_t>(p, a->partial_blocks, st);
}
