// Chunk-local gradients of the gated delta rule: one workgroup per (sequence, head, chunk).
//
// What the reference's training step gets from fla's backward of chunk_gated_delta_rule
// (lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:194-209), once the two sweeps
// over the chunks have delivered, per chunk, the state it starts from (S0), the gradient of the state it ends
// with (dS1), V~ and Y = T^T dV~.  With C = 64 tokens, gamma the prefix sum of g inside the chunk,
// e = exp(gamma), tail = exp(gamma_C - gamma), E_ij = exp(gamma_i - gamma_j) (j <= i), Q already normalised and
// scaled, K normalised:
//
//     QK = Q K^T        KK = K K^T        DP = dO V~^T        DA = Y V~^T                (64 x 64)
//     P  = tril(E . QK)                   A  = stril(beta_i E . KK)
//     dP = tril(DP)     G = dP . E        dA = -stril(DA)     Hm = dA . beta_i E
//     dQe = dO S0^T     Z  = Y S0^T       dKd = V~ dS1^T                                 (64 x K)
//     dQ  = G K + diag(e) dQe
//     dK  = G^T Q + diag(tail) dKd - diag(beta e) Z + (Hm + Hm^T) K
//     dbeta_i  = -e_i <Z_i, K_i> + <Y_i, V_i> + sum_j (dA . E . KK)_ij
//     dgamma_i = rowsum(dP . P + dA . A)_i - colsum(dP . P + dA . A)_i
//                + e_i <dQe_i, Q_i> - tail_i <dKd_i, K_i> - beta_i e_i <Z_i, K_i>
//     dgamma_C += exp(gamma_C) <dS1, S0> + sum_i tail_i <dKd_i, K_i>
//
// Every matrix product is an "A B^T" of two row-major bf16 matrices staged in LDS (the transposes of Q and K
// are staged next to them), on 32x32x16 MFMA with fp32 accumulation.  The 64 x K results are kept transposed
// ([key dim][token]) so that a lane owns one token: the per-token scales are per-lane scalars and the sums
// over the key dim stay inside a lane.  Built for K = V = 128 (157 KiB of LDS: one workgroup per CU).
#include <hip/hip_runtime.h>

#include "gdn_chunk_common.h"
#include "gdn_launch.h"

namespace gdn {

namespace {

constexpr int BWD_K = 128, BWD_V = 128;
constexpr int BWD_THREADS = 256;
constexpr int LDR = 136;  // bf16 per LDS row of a [.][128] matrix: 16 bytes of padding
constexpr int LDS64 = 72;  // bf16 per LDS row of a [.][64] matrix

struct ChunkLocalParams {
    const float* qs;
    const float* kn;
    const float* v;
    const float* dout;
    const float* y;
    const float* vnew;
    const float* s0;
    const float* ds1;
    const float* gam;
    const float* beta;
    const float* rq;  // 1 / |q|, 1 / |k| per token when q and k were normalised, else NULL
    const float* rk;
    float scale;
    float* dq;
    float* dk;
    float* dbeta;
    float* dgam;
};

// acc[r] += sum_k A[8 (r/4) + 4 h + r%4][k] B[l32][k] over k < kd: A, B point at the first of 32 rows
__device__ __forceinline__ f32x16 mma_nt(const bf16_t* A, int lda, const bf16_t* B, int ldb, int kd, f32x16 acc, int l32, int lh) {
    for (int kk = 0; kk < kd; kk += 16) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(A + l32 * lda + kk + 8 * lh);
        const bf16x8 b = *reinterpret_cast<const bf16x8*>(B + l32 * ldb + kk + 8 * lh);
        acc = mfma32_bf16(a, b, acc);
    }
    return acc;
}

// sum over the 32 lanes of a wave half, result in all of them
__device__ __forceinline__ float half_sum(float x) {
#pragma unroll
    for (int off = 16; off >= 1; off >>= 1) x += __shfl_xor(x, off, WAVE);
    return x;
}

__global__ __launch_bounds__(BWD_THREADS) void chunk_local_grads_kernel(const ChunkLocalParams p) {
    constexpr int K = BWD_K, V = BWD_V;
    __shared__ __attribute__((aligned(16))) bf16_t sQ[C * LDR];
    __shared__ __attribute__((aligned(16))) bf16_t sK[C * LDR];
    __shared__ __attribute__((aligned(16))) bf16_t sQT[K * LDS64];
    __shared__ __attribute__((aligned(16))) bf16_t sKT[K * LDS64];
    __shared__ __attribute__((aligned(16))) bf16_t sDO[C * LDR];
    __shared__ __attribute__((aligned(16))) bf16_t sVN[C * LDR];
    __shared__ __attribute__((aligned(16))) bf16_t sY[C * LDR];
    __shared__ __attribute__((aligned(16))) bf16_t sST[K * LDR];  // S0, then dS1, then G | G^T | Hm + Hm^T
    __shared__ float s_gam[C], s_beta[C], s_e[C], s_tail[C], s_dgam[C], s_dbeta[C], s_dotq[C], s_dotk[C], s_red[4];
    bf16_t* const sG = sST;
    bf16_t* const sGT = sST + C * LDS64;
    bf16_t* const sH = sST + 2 * C * LDS64;

    const int t = threadIdx.x;
    const int lane = t % WAVE, wave = t / WAVE;
    const int l32 = lane % 32, lh = lane / 32;
    const int64_t chunk = blockIdx.x;
    const float* qs = p.qs + chunk * C * K;
    const float* kn = p.kn + chunk * C * K;
    const float* vv = p.v + chunk * C * V;
    const float* dout = p.dout + chunk * C * V;
    const float* yy = p.y + chunk * C * V;
    const float* vnew = p.vnew + chunk * C * V;
    const float* s0 = p.s0 + chunk * K * V;
    const float* ds1 = p.ds1 + chunk * K * V;

    // ---- stage everything but the states ----
    if (t < C) {
        const float g = p.gam[chunk * C + t];
        s_gam[t] = g;
        s_beta[t] = p.beta[chunk * C + t];
        s_e[t] = __expf(g);
        s_tail[t] = __expf(p.gam[chunk * C + C - 1] - g);
        s_dgam[t] = 0.f;
        s_dbeta[t] = 0.f;
        s_dotq[t] = 0.f;
        s_dotk[t] = 0.f;
    }
    if (t < 4) s_red[t] = 0.f;
    auto put4 = [](bf16_t* dst, f32x4 x) {
        bf16x4 r;
        r.x = (bf16_t)x.x, r.y = (bf16_t)x.y, r.z = (bf16_t)x.z, r.w = (bf16_t)x.w;
        *reinterpret_cast<bf16x4*>(dst) = r;
    };
    float yv[8];  // <Y_i, V_i> pieces, reduced after the barrier (s_dbeta is being cleared above)
#pragma unroll
    for (int i = 0; i < 8; i++) {  // [64][128] fp32: 2048 groups of 4, row = 8 i + t / 32
        const int idx = t + BWD_THREADS * i, row = idx / 32, c4 = idx % 32;
        const f32x4 a = *reinterpret_cast<const f32x4*>(qs + row * K + 4 * c4);
        const f32x4 b = *reinterpret_cast<const f32x4*>(kn + row * K + 4 * c4);
        put4(sQ + row * LDR + 4 * c4, a);
        put4(sK + row * LDR + 4 * c4, b);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            sQT[(4 * c4 + e) * LDS64 + row] = (bf16_t)a[e];
            sKT[(4 * c4 + e) * LDS64 + row] = (bf16_t)b[e];
        }
        const f32x4 d = *reinterpret_cast<const f32x4*>(dout + row * V + 4 * c4);
        const f32x4 n = *reinterpret_cast<const f32x4*>(vnew + row * V + 4 * c4);
        const f32x4 y = *reinterpret_cast<const f32x4*>(yy + row * V + 4 * c4);
        const f32x4 x = *reinterpret_cast<const f32x4*>(vv + row * V + 4 * c4);
        put4(sDO + row * LDR + 4 * c4, d);
        put4(sVN + row * LDR + 4 * c4, n);
        put4(sY + row * LDR + 4 * c4, y);
        yv[i] = y.x * x.x + y.y * x.y + y.z * x.z + y.w * x.w;
    }
#pragma unroll
    for (int i = 0; i < 16; i++) {  // S0 [128][128] fp32: row = 8 i + t / 32
        const int idx = t + BWD_THREADS * i, row = idx / 32, c4 = idx % 32;
        put4(sST + row * LDR + 4 * c4, *reinterpret_cast<const f32x4*>(s0 + row * V + 4 * c4));
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; i++) {  // the 32 lanes of a wave half hold one row
        const float s = half_sum(yv[i]);
        if (l32 == 0) atomicAdd(&s_dbeta[8 * i + t / 32], s);
    }

    f32x16 zero;
#pragma unroll
    for (int r = 0; r < 16; r++) zero[r] = 0.f;

    // ---- products with S0, transposed: rows = key dims 32 wave .., columns = tokens 32 tt + l32 ----
    f32x16 dQeT[2], ZT[2], dKdT[2];
#pragma unroll
    for (int tt = 0; tt < 2; tt++) {
        dQeT[tt] = mma_nt(sST + 32 * wave * LDR, LDR, sDO + 32 * tt * LDR, LDR, V, zero, l32, lh);
        ZT[tt] = mma_nt(sST + 32 * wave * LDR, LDR, sY + 32 * tt * LDR, LDR, V, zero, l32, lh);
    }
    __syncthreads();  // S0 has been read by every wave

    // ---- dS1 takes the place of S0; <dS1, S0> on the way ----
    {
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int idx = t + BWD_THREADS * i, row = idx / 32, c4 = idx % 32;
            const f32x4 x = *reinterpret_cast<const f32x4*>(ds1 + row * V + 4 * c4);
            const bf16x4 s = *reinterpret_cast<const bf16x4*>(sST + row * LDR + 4 * c4);
            dot += x.x * (float)s.x + x.y * (float)s.y + x.z * (float)s.z + x.w * (float)s.w;
            put4(sST + row * LDR + 4 * c4, x);
        }
        dot = wave_sum(dot);
        if (lane == 0) atomicAdd(&s_red[0], dot);
    }
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < 2; tt++) dKdT[tt] = mma_nt(sST + 32 * wave * LDR, LDR, sVN + 32 * tt * LDR, LDR, V, zero, l32, lh);
    __syncthreads();  // the state's region is free

    // ---- the 64 x 64 products: wave -> tile (ti, tj); rows i = 32 ti + 8 (r/4) + 4 h + r%4, column j = 32 tj + l32 ----
    {
        const int ti = wave / 2, tj = wave % 2;
        const f32x16 QK = mma_nt(sQ + 32 * ti * LDR, LDR, sK + 32 * tj * LDR, LDR, K, zero, l32, lh);
        const f32x16 KK = mma_nt(sK + 32 * ti * LDR, LDR, sK + 32 * tj * LDR, LDR, K, zero, l32, lh);
        const f32x16 DP = mma_nt(sDO + 32 * ti * LDR, LDR, sVN + 32 * tj * LDR, LDR, V, zero, l32, lh);
        const f32x16 DA = mma_nt(sY + 32 * ti * LDR, LDR, sVN + 32 * tj * LDR, LDR, V, zero, l32, lh);
        const int j = 32 * tj + l32;
        const float gj = s_gam[j];
        float colsum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int i = 32 * ti + 8 * (r / 4) + 4 * lh + r % 4;
            const float bi = s_beta[i];
            const float E = i >= j ? __expf(s_gam[i] - gj) : 0.f;
            const float dP = i >= j ? DP[r] : 0.f;
            const float dA = i > j ? -DA[r] : 0.f;
            const float Pm = E * QK[r];
            const float Am = i > j ? bi * E * KK[r] : 0.f;
            const float G = dP * E;
            const float Hm = dA * bi * E;
            const float m = dP * Pm + dA * Am;
            colsum += m;
            const float rowm = half_sum(m);
            const float rowb = half_sum(dA * E * KK[r]);
            if (l32 == 0) {
                atomicAdd(&s_dgam[i], rowm);
                atomicAdd(&s_dbeta[i], rowb);
            }
            sG[i * LDS64 + j] = (bf16_t)G;
            sGT[j * LDS64 + i] = (bf16_t)G;
            if (i > j) {
                sH[i * LDS64 + j] = (bf16_t)Hm;
                sH[j * LDS64 + i] = (bf16_t)Hm;
            } else if (i == j) {
                sH[i * LDS64 + i] = (bf16_t)0.f;
            }
        }
        atomicAdd(&s_dgam[j], -colsum);
    }
    __syncthreads();

    // ---- per-token sums over the key dim, then dQ^T and dK^T ----
    float nkd = 0.f;
    f32x16 accq[2], acck[2];
#pragma unroll
    for (int tt = 0; tt < 2; tt++) {
        const int i = 32 * tt + l32;
        const float ei = s_e[i], tl = s_tail[i], bi = s_beta[i];
        float s_qe = 0.f, s_kd = 0.f, s_zk = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int d = 32 * wave + 8 * (r / 4) + 4 * lh + r % 4;
            const float qv = (float)sQT[d * LDS64 + i], kv = (float)sKT[d * LDS64 + i];
            s_qe += dQeT[tt][r] * qv;
            s_kd += dKdT[tt][r] * kv;
            s_zk += ZT[tt][r] * kv;
        }
        atomicAdd(&s_dgam[i], ei * s_qe - tl * s_kd - bi * ei * s_zk);
        atomicAdd(&s_dbeta[i], -ei * s_zk);
        nkd += tl * s_kd;

#pragma unroll
        for (int r = 0; r < 16; r++) {
            accq[tt][r] = dQeT[tt][r] * ei;
            acck[tt][r] = dKdT[tt][r] * tl - ZT[tt][r] * (bi * ei);
        }
        accq[tt] = mma_nt(sKT + 32 * wave * LDS64, LDS64, sG + 32 * tt * LDS64, LDS64, C, accq[tt], l32, lh);
        acck[tt] = mma_nt(sQT + 32 * wave * LDS64, LDS64, sGT + 32 * tt * LDS64, LDS64, C, acck[tt], l32, lh);
        acck[tt] = mma_nt(sKT + 32 * wave * LDS64, LDS64, sH + 32 * tt * LDS64, LDS64, C, acck[tt], l32, lh);
        if (p.rq != nullptr) {  // <dQs_i, Qs_i> and <dK_i, K_i> for the backward of the normalisation
            float dq_q = 0.f, dk_k = 0.f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int d = 32 * wave + 8 * (r / 4) + 4 * lh + r % 4;
                dq_q += accq[tt][r] * (float)sQT[d * LDS64 + i];
                dk_k += acck[tt][r] * (float)sKT[d * LDS64 + i];
            }
            atomicAdd(&s_dotq[i], dq_q);
            atomicAdd(&s_dotk[i], dk_k);
        }
    }
    nkd = wave_sum(nkd);
    if (lane == 0) atomicAdd(&s_red[1], nkd);
    __syncthreads();

    // With x = y / r the normalised row (y: input, r = |y|^-1 incl. epsilon): dy = r (dx - x <x, dx>); the scale of
    // q moves through: Qs = scale Qn, so dQn = scale dQs and Qn <Qn, dQn> = Qs <Qs, dQs> / scale.
#pragma unroll
    for (int tt = 0; tt < 2; tt++) {
        const int i = 32 * tt + l32;
        float* dq = p.dq + (chunk * C + i) * K + 32 * wave + 4 * lh;
        float* dk = p.dk + (chunk * C + i) * K + 32 * wave + 4 * lh;
        const bool norm = p.rq != nullptr;
        const float rq = norm ? p.rq[chunk * C + i] : 1.f, rk = norm ? p.rk[chunk * C + i] : 1.f;
        const float cq = norm ? s_dotq[i] / p.scale : 0.f, ck = norm ? s_dotk[i] : 0.f;
#pragma unroll
        for (int r4 = 0; r4 < 4; r4++) {
            f32x4 oq, ok;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int r = 4 * r4 + e, d = 32 * wave + 8 * r4 + 4 * lh + e;
                oq[e] = rq * (accq[tt][r] * p.scale - cq * (float)sQT[d * LDS64 + i]);
                ok[e] = rk * (acck[tt][r] - ck * (float)sKT[d * LDS64 + i]);
            }
            *reinterpret_cast<f32x4*>(dq + 8 * r4) = oq;
            *reinterpret_cast<f32x4*>(dk + 8 * r4) = ok;
        }
    }

    if (t < C) {
        float dg = s_dgam[t];
        if (t == C - 1) dg += s_e[C - 1] * s_red[0] + s_red[1];
        p.dgam[chunk * C + t] = dg;
        p.dbeta[chunk * C + t] = s_dbeta[t];
    }
}

}  // namespace

int launch_chunk_bwd_local(const gdn_chunk_local_args& a, hipStream_t stream) {
    ChunkLocalParams p;
    p.qs = a.qs, p.kn = a.kn, p.v = a.v, p.dout = a.dout, p.y = a.y, p.vnew = a.v_new;
    p.s0 = a.states, p.ds1 = a.dstates, p.gam = a.gamma, p.beta = a.beta;
    p.rq = a.rq, p.rk = a.rk, p.scale = a.scale;
    p.dq = a.dq, p.dk = a.dk, p.dbeta = a.dbeta, p.dgam = a.dgamma;
    hipLaunchKernelGGL(chunk_local_grads_kernel, dim3((unsigned)a.chunks), dim3(BWD_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}

bool chunk_bwd_local_supported(const gdn_chunk_local_args& a) { return a.K == BWD_K && a.V == BWD_V; }

}  // namespace gdn
