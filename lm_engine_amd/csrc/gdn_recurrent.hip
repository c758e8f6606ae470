// Token-by-token gated delta rule with the state tile resident in registers.
//
// One workgroup of 256 threads owns the K x BV tile of one (sequence, head) state: columns
// of the state evolve independently, so V is split over workgroups without any exchange.
// Each thread holds RPT consecutive rows x 4 consecutive columns (fp32) of the tile; a wave's
// loads are whole 16 B-per-lane rows of the tile.  Per token:
//
//     r  = beta (v - e^g S^T k)        S' = e^g S + k r^T        o = e^g S^T q + (k . q) r
//
// i.e. one read and one write of the state for T == 1 (the decode step); both are streaming
// (non-temporal) accesses, since a state far larger than the caches is touched exactly once per step.  The two
// K-reductions (S^T k, S^T q) are done in registers, then across the row groups of a wave
// with shuffles and across the four waves through LDS.
//
// Replaces fla.ops.gated_delta_rule.fused_recurrent_gated_delta_rule as called at
// lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:210-222.

#include "gdn_common.h"
#include "gdn_launch.h"

namespace gdn {

constexpr int REC_THREADS = 256;
constexpr int REC_WAVES = REC_THREADS / WAVE;

struct RecurrentParams {
    const void* q;
    const void* k;
    const void* v;
    const void* beta;
    const float* g;
    const float* h0;
    float* ht;
    void* o;
    const int32_t* cu_seqlens;
    const int32_t* pad_lens;  // left-padded batch: prefix sums of the valid lengths
    int64_t q_stride_b, q_stride_t, q_stride_h;
    int64_t k_stride_b, k_stride_t, k_stride_h;
    int64_t v_stride_b, v_stride_t, v_stride_h;
    int64_t o_stride_b, o_stride_t, o_stride_h;
    int T, H, V;
    int qk_div;  // value heads per head of q and k
    int beta_dtype;
    int l2norm;
    float scale;
};

template <typename T, int K, int BV>
__global__ __launch_bounds__(REC_THREADS) void recurrent_kernel(const RecurrentParams p) {
    constexpr int LANES_V = BV / 4;            // lanes along the value dim (4 columns each)
    constexpr int ROWG = REC_THREADS / LANES_V;  // row groups in the workgroup
    constexpr int RPT = K / ROWG;              // state rows per thread
    constexpr int KPL = K / WAVE;  // q/k elements per lane when one wave loads a whole row
    static_assert(K % ROWG == 0 && RPT >= 1, "tile does not divide over the workgroup");
    static_assert(K % WAVE == 0, "K must be a multiple of the wave size");

    // k^ is read again after the second barrier of a token (the rank-1 update) while wave 0 may already be
    // staging the next token: two buffers, alternating by token.  q^ and k^ . q^ are only read between the
    // two barriers, where wave 0 cannot have moved on.
    __shared__ __attribute__((aligned(16))) float s_k2[2][K];
    __shared__ __attribute__((aligned(16))) float s_q[K];
    __shared__ float s_kq[1];
    __shared__ __attribute__((aligned(16))) float s_red[REC_WAVES][LANES_V][8];

    const int tid = threadIdx.x;
    const int lane = tid % WAVE;
    const int wave = tid / WAVE;
    const int lv = tid % LANES_V;   // which 4 columns
    const int rg = tid / LANES_V;   // which row group
    const int v0 = blockIdx.x * BV + lv * 4;
    const int h = blockIdx.y;
    const int n = blockIdx.z;

    int64_t b = n, t_begin = 0, t_end = p.T;
    if (p.pad_lens != nullptr) t_begin = p.T - min(max(p.pad_lens[n + 1] - p.pad_lens[n], 0), p.T);  // the last tokens of row n
    if (p.cu_seqlens != nullptr) {
        int t0, len;
        packed_bounds(p.cu_seqlens, n, p.T, t0, len);
        b = 0, t_begin = t0, t_end = t0 + len;
    }

    const int64_t state_off = (((int64_t)n * p.H + h) * K + (int64_t)rg * RPT) * p.V + v0;

    f32x4 S[RPT];
    if (p.h0 != nullptr) {
#pragma unroll
        for (int i = 0; i < RPT; i++) S[i] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p.h0 + state_off + (int64_t)i * p.V));
    } else {
#pragma unroll
        for (int i = 0; i < RPT; i++) S[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    const int64_t hqk = p.qk_div > 1 ? h / p.qk_div : h;
    const T* qp = reinterpret_cast<const T*>(p.q) + b * p.q_stride_b + hqk * p.q_stride_h;
    const T* kp = reinterpret_cast<const T*>(p.k) + b * p.k_stride_b + hqk * p.k_stride_h;
    const T* vp = reinterpret_cast<const T*>(p.v) + b * p.v_stride_b + h * p.v_stride_h + v0;
    T* op = reinterpret_cast<T*>(p.o) + b * p.o_stride_b + h * p.o_stride_h + v0;

    for (int64_t t = t_begin; t < t_end; t++) {
        float* const s_k = s_k2[(t - t_begin) & 1];
        // ---- wave 0 stages k^ and q^ (normalised, q scaled) in LDS; others go straight on ----
        if (wave == 0) {
            float kx[KPL], qx[KPL];
            float ssk = 0.f, ssq = 0.f;
#pragma unroll
            for (int e = 0; e < KPL; e++) {
                kx[e] = to_f32(kp[t * p.k_stride_t + lane * KPL + e]);
                qx[e] = to_f32(qp[t * p.q_stride_t + lane * KPL + e]);
                ssk += kx[e] * kx[e];
                ssq += qx[e] * qx[e];
            }
            float kn = 1.f, qn = p.scale;
            if (p.l2norm) {
                kn = rsqrtf(wave_sum(ssk) + L2NORM_EPS);
                qn = rsqrtf(wave_sum(ssq) + L2NORM_EPS) * p.scale;
            }
            float kq = 0.f;
#pragma unroll
            for (int e = 0; e < KPL; e++) {
                kx[e] *= kn;
                qx[e] *= qn;
                kq += kx[e] * qx[e];
                s_k[lane * KPL + e] = kx[e];
                s_q[lane * KPL + e] = qx[e];
            }
            kq = wave_sum(kq);
            if (lane == 0) s_kq[0] = kq;
        }
        const int64_t sidx = (b * p.T + t) * p.H + h;
        const float eg = (p.g != nullptr) ? expf(p.g[sidx]) : 1.0f;
        const float beta = load_beta(p.beta, p.beta_dtype, sidx);
        const f32x4 vt = load4<T>(vp + t * p.v_stride_t);
        __syncthreads();

        // ---- partial S^T k and S^T q over this thread's rows ----
        f32x4 pk = {0.f, 0.f, 0.f, 0.f}, pq = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < RPT; i++) {
            const float kr = s_k[rg * RPT + i];
            const float qr = s_q[rg * RPT + i];
            pk += S[i] * kr;
            pq += S[i] * qr;
        }
        const float kq = s_kq[0];
        // row groups inside a wave
#pragma unroll
        for (int off = LANES_V; off < WAVE; off <<= 1) {
#pragma unroll
            for (int c = 0; c < 4; c++) {
                pk[c] += __shfl_xor(pk[c], off, WAVE);
                pq[c] += __shfl_xor(pq[c], off, WAVE);
            }
        }
        if (lane < LANES_V) {
            *reinterpret_cast<f32x4*>(&s_red[wave][lane][0]) = pk;
            *reinterpret_cast<f32x4*>(&s_red[wave][lane][4]) = pq;
        }
        __syncthreads();
        f32x4 sk = {0.f, 0.f, 0.f, 0.f}, sq = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < REC_WAVES; w++) {
            sk += *reinterpret_cast<const f32x4*>(&s_red[w][lv][0]);
            sq += *reinterpret_cast<const f32x4*>(&s_red[w][lv][4]);
        }

        // ---- rank-1 update and output ----
        const f32x4 r = (vt - sk * eg) * beta;
#pragma unroll
        for (int i = 0; i < RPT; i++) S[i] = S[i] * eg + r * s_k[rg * RPT + i];  // k^ re-read: keeps 16 registers free
        if (rg == 0) store4<T>(op + t * p.o_stride_t, sq * eg + r * kq);
    }

    if (p.ht != nullptr) {
#pragma unroll
        for (int i = 0; i < RPT; i++) __builtin_nontemporal_store(S[i], reinterpret_cast<f32x4*>(p.ht + state_off + (int64_t)i * p.V));
    }
}

template <typename T, int K, int BV>
static int launch_recurrent_tile(const RecurrentParams& p, int N, hipStream_t stream) {
    dim3 grid(p.V / BV, p.H, N);
    hipLaunchKernelGGL((recurrent_kernel<T, K, BV>), grid, dim3(REC_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}

template <typename T, int K>
static int launch_recurrent_k(const RecurrentParams& p, int N, hipStream_t stream) {
    // Wide tiles give the longest contiguous rows; narrow ones give more workgroups when
    // there are few (sequence, head) pairs.
    const int64_t pairs = (int64_t)N * p.H;
    if constexpr (K <= 128) {  // a K = 256 tile of 128 columns would not fit the register file
        if (p.V % 128 == 0 && pairs * (p.V / 128) >= 1024) return launch_recurrent_tile<T, K, 128>(p, N, stream);
    }
    if (p.V % 64 == 0 && pairs * (p.V / 64) >= 512) return launch_recurrent_tile<T, K, 64>(p, N, stream);
    return launch_recurrent_tile<T, K, 32>(p, N, stream);
}

template <typename T>
static int launch_recurrent_t(const RecurrentParams& p, int K, int N, hipStream_t stream) {
    switch (K) {
        case 64: return launch_recurrent_k<T, 64>(p, N, stream);
        case 128: return launch_recurrent_k<T, 128>(p, N, stream);
        case 256: return launch_recurrent_k<T, 256>(p, N, stream);
        default: return GDN_ERR_UNSUPPORTED;
    }
}

int launch_recurrent(const gdn_args& a, hipStream_t stream) {
    RecurrentParams p;
    p.q = a.q;
    p.k = a.k;
    p.v = a.v;
    p.beta = a.beta;
    p.g = a.g;
    p.h0 = a.h0;
    p.ht = a.ht;
    p.o = a.o;
    p.cu_seqlens = (a.flags & GDN_FLAG_LEFT_PADDED) ? nullptr : a.cu_seqlens;
    p.pad_lens = (a.flags & GDN_FLAG_LEFT_PADDED) ? a.cu_seqlens : nullptr;
    p.q_stride_b = a.q_stride_b, p.q_stride_t = a.q_stride_t, p.q_stride_h = a.q_stride_h;
    p.k_stride_b = a.k_stride_b, p.k_stride_t = a.k_stride_t, p.k_stride_h = a.k_stride_h;
    p.v_stride_b = a.v_stride_b, p.v_stride_t = a.v_stride_t, p.v_stride_h = a.v_stride_h;
    p.o_stride_b = a.o_stride_b, p.o_stride_t = a.o_stride_t, p.o_stride_h = a.o_stride_h;
    p.T = a.T, p.H = a.H, p.V = a.V;
    p.qk_div = a.qk_heads > 0 ? a.H / a.qk_heads : 1;
    p.beta_dtype = a.beta_dtype;
    p.l2norm = (a.flags & GDN_FLAG_L2NORM) ? 1 : 0;
    p.scale = a.scale;
    if (a.dtype == GDN_BF16) return launch_recurrent_t<bf16_t>(p, a.K, a.N, stream);
    if (a.dtype == GDN_F32) return launch_recurrent_t<float>(p, a.K, a.N, stream);
    return GDN_ERR_UNSUPPORTED;
}

}  // namespace gdn
