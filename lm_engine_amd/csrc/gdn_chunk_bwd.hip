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
// over the key dim stay inside a lane.  Built for K = 128 and V = 128, 256 or 512 (the value dim is staged 128 columns
// at a time; 157 KiB of LDS: one workgroup per CU).
#include <hip/hip_runtime.h>

#include "gdn_chunk_common.h"
#include "gdn_launch.h"

namespace gdn {

namespace {

constexpr int BWD_K = 128;  // the kernels of this file are built for K = 128 and V = 128, 256 or 512
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
    // "final" mode (whole-chunk batches; chunk = (n H + h) NC + c): Y is read from the output of the scan over
    // the mirror problem, and the gradients go out in the caller's layout, [N, NC 64, H, .] bf16 for q, k, v and
    // fp32 [N, NC 64, H] for g (reverse prefix sum of dgamma done here) and beta
    const bf16_t* y_mirror;  // [N][2 NC 64][H][V], NULL = packed mode
    // final mode reads the caller's q, k, v, dO (bf16, element strides) instead of the packed qs, kn, v, dout
    const bf16_t* q_raw;
    const bf16_t* k_raw;
    const bf16_t* v_raw;
    const bf16_t* d_raw;
    int64_t q_stride_b, q_stride_t, q_stride_h;
    int64_t k_stride_b, k_stride_t, k_stride_h;
    int64_t v_stride_b, v_stride_t, v_stride_h;
    int64_t d_stride_b, d_stride_t, d_stride_h;
    bf16_t* dq_out;
    bf16_t* dk_out;
    bf16_t* dv_out;
    float* dg_out;
    float* dbeta_out;
    int H, NC;
    // sequences that are not whole rows of whole chunks (packed or left-padded batches): first token (flat index
    // over the rows of the caller's tensors) and length of every sequence; NULL = sequence n is row n
    const int32_t* seq_start;
    const int32_t* seq_len;
    int T_rows;  // tokens per row of the caller's tensors
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

template <int V>
__global__ __launch_bounds__(BWD_THREADS) void chunk_local_grads_kernel(const ChunkLocalParams p) {
    constexpr int K = BWD_K, VW = 128;  // VW: columns of the value dim staged at a time
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
    const float* qs = p.qs + chunk * C * K;  // packed mode only
    const float* kn = p.kn + chunk * C * K;
    const float* vv = p.v + chunk * C * V;
    const float* dout = p.dout + chunk * C * V;
    const bool final_mode = p.y_mirror != nullptr;
    const int ci = final_mode ? (int)(chunk % p.NC) : 0;
    const int chain = final_mode ? (int)(chunk / p.NC) : 0;
    const int n = final_mode ? chain / p.H : 0, h = final_mode ? chain % p.H : 0;
    // first token of the chunk as a flat index over the rows of the caller's tensors, and its number of tokens
    int valid = C;
    int64_t tok0 = 0;
    if (final_mode) {
        if (p.seq_start != nullptr) {
            valid = min(max(p.seq_len[n] - ci * C, 0), C);
            tok0 = (int64_t)p.seq_start[n] + (int64_t)ci * C;
        } else {
            tok0 = (int64_t)n * p.T_rows + (int64_t)ci * C;
        }
        if (valid == 0) return;  // a chunk past the end of its sequence (whole workgroup)
    }
    const int64_t mirA = ((int64_t)n * p.NC + (p.NC - 1 - ci)) * 2 * C;  // first token of mirror chunk A
    // row `row` of the chunk in one of the caller's tensors; rows past the end read token 0 and are zeroed
    auto row_of = [&](const bf16_t* base, int64_t sb, int64_t st, int64_t sh, int row) -> const bf16_t* {
        const int64_t f = row < valid ? tok0 + row : 0;
        return base + (f / p.T_rows) * sb + (f % p.T_rows) * st + (int64_t)h * sh;
    };
    bf16x8 zero8;
#pragma unroll
    for (int e = 0; e < 8; e++) zero8[e] = (bf16_t)0.f;
    const float* yy = final_mode ? nullptr : p.y + chunk * C * V;
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
    // ---- q, k and their transposes (final mode: with the first half of v, dO, Y below, one batch of loads) ----
    if (!final_mode) {
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
        }
    }

    f32x16 zero;
#pragma unroll
    for (int r = 0; r < 16; r++) zero[r] = 0.f;

    // Everything that contracts over the value dim runs over V in halves of 128 columns (VW), accumulating:
    // the products with the states, transposed (rows = key dims 32 wave .., columns = tokens 32 tt + l32), and
    // the 64 x 64 products dO V~^T and Y V~^T (wave -> tile (wave / 2, wave % 2)).
    f32x16 dQeT[2] = {zero, zero}, ZT[2] = {zero, zero}, dKdT[2] = {zero, zero}, DP = zero, DA = zero;
#pragma unroll
    for (int hv = 0; hv < V / VW; hv++) {
        const int v0 = VW * hv;
        float yv[8];  // <Y_i, V_i> pieces, reduced after the barrier (s_dbeta is cleared before the first one)
#pragma unroll
        for (int i = 0; i < 8; i++) yv[i] = 0.f;
        if (final_mode) {
            // v, dO and Y (token `row` is token 63 - row of mirror chunk A); dV = beta Y goes out right away
            const int p8 = t % 16;
#pragma unroll
            for (int it = 0; it < 4; it++) {
                const int row = t / 16 + 16 * it;
                const bool live = row < valid;
                if (hv == 0) {
                    bf16x8 qr = *reinterpret_cast<const bf16x8*>(row_of(p.q_raw, p.q_stride_b, p.q_stride_t, p.q_stride_h, row) + 8 * p8);
                    bf16x8 kr = *reinterpret_cast<const bf16x8*>(row_of(p.k_raw, p.k_stride_b, p.k_stride_t, p.k_stride_h, row) + 8 * p8);
                    if (!live) qr = zero8, kr = zero8;
                    const float fq = (p.rq != nullptr ? p.rq[chunk * C + row] : 1.f) * p.scale;
                    const float fk = p.rk != nullptr ? p.rk[chunk * C + row] : 1.f;
                    bf16x8 qb, kb;
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        qb[e] = (bf16_t)((float)qr[e] * fq);
                        kb[e] = (bf16_t)((float)kr[e] * fk);
                        sQT[(8 * p8 + e) * LDS64 + row] = qb[e];
                        sKT[(8 * p8 + e) * LDS64 + row] = kb[e];
                    }
                    *reinterpret_cast<bf16x8*>(sQ + row * LDR + 8 * p8) = qb;
                    *reinterpret_cast<bf16x8*>(sK + row * LDR + 8 * p8) = kb;
                }
                bf16x8 vr = *reinterpret_cast<const bf16x8*>(row_of(p.v_raw, p.v_stride_b, p.v_stride_t, p.v_stride_h, row) + v0 + 8 * p8);
                bf16x8 dr = *reinterpret_cast<const bf16x8*>(row_of(p.d_raw, p.d_stride_b, p.d_stride_t, p.d_stride_h, row) + v0 + 8 * p8);
                if (!live) vr = zero8, dr = zero8;
                const bf16x8 yr = *reinterpret_cast<const bf16x8*>(p.y_mirror + ((mirA + (C - 1 - row)) * p.H + h) * V + v0 + 8 * p8);
                const float b = p.beta[chunk * C + row];
                bf16x8 dv;
                float acc = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    dv[e] = (bf16_t)((float)yr[e] * b);
                    acc += (float)yr[e] * (float)vr[e];
                }
                *reinterpret_cast<bf16x8*>(sDO + row * LDR + 8 * p8) = dr;
                *reinterpret_cast<bf16x8*>(sY + row * LDR + 8 * p8) = yr;
                if (live) *reinterpret_cast<bf16x8*>(p.dv_out + ((tok0 + row) * p.H + h) * V + v0 + 8 * p8) = dv;
                yv[it] = acc;
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {  // rows of V~ past the end of the sequence hold whatever the scan left
                const int idx = t + BWD_THREADS * i, row = idx / 32, c4 = idx % 32;
                const f32x4 x = *reinterpret_cast<const f32x4*>(vnew + row * V + v0 + 4 * c4);
                put4(sVN + row * LDR + 4 * c4, row < valid ? x : f32x4{0.f, 0.f, 0.f, 0.f});
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int idx = t + BWD_THREADS * i, row = idx / 32, c4 = idx % 32;
                const f32x4 d = *reinterpret_cast<const f32x4*>(dout + row * V + v0 + 4 * c4);
                const f32x4 n4 = *reinterpret_cast<const f32x4*>(vnew + row * V + v0 + 4 * c4);
                const f32x4 y = *reinterpret_cast<const f32x4*>(yy + row * V + v0 + 4 * c4);
                const f32x4 x = *reinterpret_cast<const f32x4*>(vv + row * V + v0 + 4 * c4);
                put4(sDO + row * LDR + 4 * c4, d);
                put4(sVN + row * LDR + 4 * c4, n4);
                put4(sY + row * LDR + 4 * c4, y);
                yv[i] = y.x * x.x + y.y * x.y + y.z * x.z + y.w * x.w;
            }
        }
#pragma unroll
        for (int i = 0; i < 16; i++) {  // S0[:, v0 .. v0 + 127] fp32: row = 8 i + t / 32
            const int idx = t + BWD_THREADS * i, row = idx / 32, c4 = idx % 32;
            put4(sST + row * LDR + 4 * c4, *reinterpret_cast<const f32x4*>(s0 + row * V + v0 + 4 * c4));
        }
        __syncthreads();
        if (final_mode) {
#pragma unroll
            for (int it = 0; it < 4; it++) {  // 16 lanes hold one row
                float x = yv[it];
#pragma unroll
                for (int off = 8; off >= 1; off >>= 1) x += __shfl_xor(x, off, WAVE);
                if (t % 16 == 0) atomicAdd(&s_dbeta[t / 16 + 16 * it], x);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) {  // the 32 lanes of a wave half hold one row
                const float x = half_sum(yv[i]);
                if (l32 == 0) atomicAdd(&s_dbeta[8 * i + t / 32], x);
            }
        }

        // dS1 of this half is asked for now and stays in registers while the products with S0 run: its trip through
        // memory is then behind them instead of in front of the barrier below (the workgroup has a CU to itself by its
        // LDS, so there is no other wave to fill the wait)
        f32x4 ds1_rows[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int idx = t + BWD_THREADS * i, row = idx / 32, c4 = idx % 32;
            ds1_rows[i] = *reinterpret_cast<const f32x4*>(ds1 + row * V + v0 + 4 * c4);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
            dQeT[tt] = mma_nt(sST + 32 * wave * LDR, LDR, sDO + 32 * tt * LDR, LDR, VW, dQeT[tt], l32, lh);
            ZT[tt] = mma_nt(sST + 32 * wave * LDR, LDR, sY + 32 * tt * LDR, LDR, VW, ZT[tt], l32, lh);
        }
        if constexpr (V > VW) {  // with a single half they wait until the 64 x 64 stage below (dO, V~, Y stay staged)
            DP = mma_nt(sDO + 32 * (wave / 2) * LDR, LDR, sVN + 32 * (wave % 2) * LDR, LDR, VW, DP, l32, lh);
            DA = mma_nt(sY + 32 * (wave / 2) * LDR, LDR, sVN + 32 * (wave % 2) * LDR, LDR, VW, DA, l32, lh);
        }
        __syncthreads();  // S0 has been read by every wave

        // dS1 takes the place of S0; <dS1, S0> on the way
        {
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int idx = t + BWD_THREADS * i, row = idx / 32, c4 = idx % 32;
                const f32x4 x = ds1_rows[i];
                const bf16x4 sv = *reinterpret_cast<const bf16x4*>(sST + row * LDR + 4 * c4);
                dot += x.x * (float)sv.x + x.y * (float)sv.y + x.z * (float)sv.z + x.w * (float)sv.w;
                put4(sST + row * LDR + 4 * c4, x);
            }
            dot = wave_sum(dot);
            if (lane == 0) atomicAdd(&s_red[0], dot);
        }
        __syncthreads();
#pragma unroll
        for (int tt = 0; tt < 2; tt++) dKdT[tt] = mma_nt(sST + 32 * wave * LDR, LDR, sVN + 32 * tt * LDR, LDR, VW, dKdT[tt], l32, lh);
        __syncthreads();  // the staged half is free
    }

    // ---- the 64 x 64 products: wave -> tile (ti, tj); rows i = 32 ti + 8 (r/4) + 4 h + r%4, column j = 32 tj + l32 ----
    {
        const int ti = wave / 2, tj = wave % 2;
        const f32x16 QK = mma_nt(sQ + 32 * ti * LDR, LDR, sK + 32 * tj * LDR, LDR, K, zero, l32, lh);
        const f32x16 KK = mma_nt(sK + 32 * ti * LDR, LDR, sK + 32 * tj * LDR, LDR, K, zero, l32, lh);
        if constexpr (V == VW) {
            DP = mma_nt(sDO + 32 * ti * LDR, LDR, sVN + 32 * tj * LDR, LDR, VW, zero, l32, lh);
            DA = mma_nt(sY + 32 * ti * LDR, LDR, sVN + 32 * tj * LDR, LDR, VW, zero, l32, lh);
        }
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
        const int64_t at = final_mode ? ((tok0 + i) * p.H + h) * K + 32 * wave + 4 * lh : (chunk * C + i) * K + 32 * wave + 4 * lh;
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
            if (final_mode) {
                if (i < valid) {
                    store4<bf16_t>(p.dq_out + at + 8 * r4, oq);
                    store4<bf16_t>(p.dk_out + at + 8 * r4, ok);
                }
            } else {
                *reinterpret_cast<f32x4*>(p.dq + at + 8 * r4) = oq;
                *reinterpret_cast<f32x4*>(p.dk + at + 8 * r4) = ok;
            }
        }
    }

    if (t < C) {  // wave 0
        float dg = s_dgam[t];
        if (t == C - 1) dg += s_e[C - 1] * s_red[0] + s_red[1];
        if (final_mode) {
            // dg_t = sum of dgamma over the tokens t .. 63 of the chunk
#pragma unroll
            for (int off = 1; off < WAVE; off <<= 1) {
                const float y = __shfl_down(dg, off, WAVE);
                if (t + off < C) dg += y;
            }
            if (t < valid) {
                p.dg_out[(tok0 + t) * p.H + h] = dg;
                p.dbeta_out[(tok0 + t) * p.H + h] = s_dbeta[t];
            }
        } else {
            p.dgam[chunk * C + t] = dg;
            p.dbeta[chunk * C + t] = s_dbeta[t];
        }
    }
}


// ------------------------------------------------------------------------------------------
// Everything the backward needs per chunk before its two sweeps, one workgroup per (sequence, head, chunk),
// for batches of whole chunks (one sequence per row, T a multiple of 64):
//   * gamma, beta (fp32) and the inverse norms of the rows of q and k, packed per chunk, for
//     chunk_local_grads_kernel;
//   * the "mirror" problem that turns the reverse sweep into a forward scan (tokens in reverse order; chunk c
//     becomes chunks A, B = 2 r, 2 r + 1 with r = NC - 1 - c):
//         A:  v := P^T dO, k := k, T' := T^T mirrored, P := I, row scales of k: -tail / |k| before T',
//             -beta e / |k| for the state update, e^{gamma_C} decay
//         B:  v := dO, k := q, T' := I, P := 0, row scale e scale / |q| for the state update, no decay
//     i.e. the rows of k_m and v_m and both records, in the layout chunk_prepare32_kernel writes.
// T = (I + A)^-1 is formed by forward substitution in one wave (a lane owns a column, 2016 multiply-adds).
// ------------------------------------------------------------------------------------------
constexpr int LDA = 68;  // floats per LDS row of A / T

struct BwdPrepareParams {
    const bf16_t* q;
    const bf16_t* k;
    const bf16_t* dout;
    const float* g;  // [N][T][H], NULL = 0
    const void* beta;  // [N][T][H], NULL = 1
    int beta_dtype;
    int64_t q_stride_b, q_stride_t, q_stride_h;
    int64_t k_stride_b, k_stride_t, k_stride_h;
    int64_t d_stride_b, d_stride_t, d_stride_h;
    int N, H, NC;
    int l2norm;
    int rec16;  // fragments of the records in the lane order of the 16x16x32 MFMA (GDN_FLAG_RECORDS_16X16)
    float scale;
    float* gam;
    float* bc;
    float* rq;
    float* rk;
    const int32_t* seq_start;  // as in ChunkLocalParams
    const int32_t* seq_len;
    int T_rows;
    bf16_t* k_m;
    bf16_t* v_m;
    uint8_t* rec;
    uint32_t rec_bytes, off_p, off_qs, off_ks, off_cs, off_eg;
};

// T = (I + A)^-1 for a strictly lower-triangular 64 x 64 matrix A (fp32 in LDS, rows LDA floats apart, zeros on and
// above the diagonal), in place, by the four waves of the workgroup together; `scratch` holds INVERSE_SCRATCH_FLOATS.
// The same blocked scheme as the forward's prepare step (gdn_chunk_prepare32.h, which interleaves it with its tile
// products): wave 0 inverts the four 16 x 16 diagonal blocks by substitution (a lane owns a column: 120 dependent
// multiply-adds instead of the 2016 of a substitution over all 64 rows), then the blocks below the diagonal follow
// from T_BA = -T_BB (A_BA T_AA), first with 16 x 16 blocks on two waves, then with 32 x 32 blocks, one 16 x 16
// output tile per wave, as products on the fp32 MFMA (16x16x4: no operand is rounded).  Ends with a barrier.
constexpr int INV_LDT = 36, INV_LDM = 20;  // floats per row of the transposed 32 x 32 and 16 x 16 scratch blocks
constexpr int INVERSE_SCRATCH_FLOATS = 32 * INV_LDT + 2 * 16 * INV_LDM + 32 * INV_LDT;
template <int LDA_>
__device__ __forceinline__ void invert_unit_lower_64(float* sA, float* scratch, const int wave, const int lane) {
    constexpr int LDT = INV_LDT, LDM = INV_LDM;
    float* const sT = sA;
    float* const sTtA = scratch;           // transpose of the top-left 32 x 32 of T
    float* const sMt = sTtA + 32 * LDT;    // transposed products of the first merge
    float* const sMtB = sMt + 2 * 16 * LDM;  // transposed product of the second merge
    const int l16 = lane % 16, lq = lane / 16;
    __syncthreads();  // A is complete and the scratch is free
    float x[16];  // column l16 of the inverse of diagonal block lq (wave 0)
    if (wave == 0) {
        const float* a = &sA[(16 * lq) * LDA_ + 16 * lq];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            f32x4 row[4];
#pragma unroll
            for (int c4 = 0; c4 < (i + 3) / 4; c4++) row[c4] = *reinterpret_cast<const f32x4*>(&a[i * LDA_ + 4 * c4]);
            float part[4] = {(i == l16) ? 1.f : 0.f, 0.f, 0.f, 0.f};  // four independent partial sums
#pragma unroll
            for (int kk = 0; kk < i; kk++) part[kk % 4] -= row[kk / 4][kk % 4] * x[kk];
            x[i] = (part[0] + part[1]) + (part[2] + part[3]);
        }
        // every lane of the wave has read its block of A by now (one wave, program order)
#pragma unroll
        for (int i = 0; i < 16; i++) sT[(16 * lq + i) * LDA_ + 16 * lq + l16] = x[i];
    }
    __syncthreads();
    // 16 x 16 output tile of a product X Y: lane (l16, lq) supplies reduction entries k = 4 n lq + e, e < 4 n, of row l16
    // of X and of column l16 of Y (a row of Y^T); MFMA e takes entry e of every lane.
    auto mm16 = [&](const float* xrow, const float* ytrow) -> f32x4 {
        const f32x4 xv = *reinterpret_cast<const f32x4*>(xrow), yv = *reinterpret_cast<const f32x4*>(ytrow);
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; e++) acc = mfma_f32(xv[e], yv[e], acc);
        return acc;
    };
    auto mm16x32 = [&](const float* xrow, const float* ytrow) -> f32x4 {
        const f32x4 x0 = *reinterpret_cast<const f32x4*>(xrow), x1 = *reinterpret_cast<const f32x4*>(xrow + 4);
        const f32x4 y0 = *reinterpret_cast<const f32x4*>(ytrow), y1 = *reinterpret_cast<const f32x4*>(ytrow + 4);
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; e++) acc = mfma_f32(x0[e], y0[e], acc);
#pragma unroll
        for (int e = 0; e < 4; e++) acc = mfma_f32(x1[e], y1[e], acc);
        return acc;
    };
    // first merge: T_10 = -T_11 (A_10 T_00) on wave 0, T_32 = -T_33 (A_32 T_22) on wave 1
    if (wave < 2) {
        const int bi = 2 * wave + 1, bj = 2 * wave;
        const int kk = 4 * lq;
        float* const mt = &sMt[wave * 16 * LDM];
        f32x4 y0;  // column l16 of T_bj,bj, entries kk .. kk + 3 (a row of its transpose)
#pragma unroll
        for (int e = 0; e < 4; e++) y0[e] = sT[(16 * bj + kk + e) * LDA_ + 16 * bj + l16];
        f32x4 m = {0.f, 0.f, 0.f, 0.f};
        {
            const f32x4 xa = *reinterpret_cast<const f32x4*>(&sA[(16 * bi + l16) * LDA_ + 16 * bj + kk]);
#pragma unroll
            for (int e = 0; e < 4; e++) m = mfma_f32(xa[e], y0[e], m);
        }
        if (wave == 0 && lq < 2) {
            // the transposes of T_00 and T_11 for the second merge, from the registers of the inverse, and the zero block (T_01)^T
#pragma unroll
            for (int c4 = 0; c4 < 4; c4++)
                *reinterpret_cast<f32x4*>(&sTtA[(16 * lq + l16) * LDT + 16 * lq + 4 * c4]) = f32x4{x[4 * c4], x[4 * c4 + 1], x[4 * c4 + 2], x[4 * c4 + 3]};
            if (lq == 1) {
#pragma unroll
                for (int c4 = 0; c4 < 4; c4++) *reinterpret_cast<f32x4*>(&sTtA[(16 + l16) * LDT + 4 * c4]) = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
        *reinterpret_cast<f32x4*>(&mt[l16 * LDM + 4 * lq]) = m;  // M^T[n][4 lq + e]
        const f32x4 t = mm16(&sT[(16 * bi + l16) * LDA_ + 16 * bi + kk], &mt[l16 * LDM + kk]);
#pragma unroll
        for (int e = 0; e < 4; e++) sT[(16 * bi + 4 * lq + e) * LDA_ + 16 * bj + l16] = -t[e];  // over A_bi,bj, read above
        if (wave == 0) *reinterpret_cast<f32x4*>(&sTtA[l16 * LDT + 16 + 4 * lq]) = -t;  // (T_10)^T
    }
    __syncthreads();
    // second merge: T_BA = -T_BB (A_BA T_AA) with 32 x 32 blocks; one 16 x 16 output tile per wave
    {
        const int ta = wave / 2, tb = wave % 2;
        const f32x4 m = mm16x32(&sA[(32 + 16 * ta + l16) * LDA_ + 8 * lq], &sTtA[(16 * tb + l16) * LDT + 8 * lq]);
        *reinterpret_cast<f32x4*>(&sMtB[(16 * tb + l16) * LDT + 16 * ta + 4 * lq]) = m;
        __syncthreads();
        const f32x4 t = mm16x32(&sT[(32 + 16 * ta + l16) * LDA_ + 32 + 8 * lq], &sMtB[(16 * tb + l16) * LDT + 8 * lq]);
#pragma unroll
        for (int e = 0; e < 4; e++) sT[(32 + 16 * ta + 4 * lq + e) * LDA_ + 16 * tb + l16] = -t[e];
    }
    __syncthreads();  // T is complete
}

template <int V>
__global__ __launch_bounds__(BWD_THREADS) void chunk_bwd_prepare_kernel(const BwdPrepareParams p) {
    constexpr int K = BWD_K;
    __shared__ __attribute__((aligned(16))) bf16_t sQ[C * LDR];
    __shared__ __attribute__((aligned(16))) bf16_t sK[C * LDR];
    __shared__ __attribute__((aligned(16))) bf16_t sDOT[V * LDS64];  // dO^T
    __shared__ __attribute__((aligned(16))) bf16_t sPT[C * LDS64];   // P^T
    __shared__ __attribute__((aligned(16))) float sA[C * LDA];       // A, then T in its place
    __shared__ float s_gam[C], s_beta[C], s_e[C], s_tail[C], s_rq[C], s_rk[C];

    const int t = threadIdx.x;
    const int lane = t % WAVE, wave = t / WAVE;
    const int l32 = lane % 32, lh = lane / 32;
    const int64_t chunk = blockIdx.x;
    const int ci = (int)(chunk % p.NC);
    const int chain = (int)(chunk / p.NC);
    const int n = chain / p.H, h = chain % p.H;
    const int64_t TM = (int64_t)p.NC * 2 * C;  // tokens per sequence of the mirror problem
    // first token of the chunk as a flat index over the rows of the caller's tensors, and its number of tokens;
    // a chunk past the end of its sequence (valid = 0) still gets its (neutral) records and zero rows
    int valid = C;
    int64_t tok0 = (int64_t)n * p.T_rows + (int64_t)ci * C;
    if (p.seq_start != nullptr) {
        valid = min(max(p.seq_len[n] - ci * C, 0), C);
        tok0 = (int64_t)p.seq_start[n] + (int64_t)ci * C;
    }
    auto row_of = [&](const bf16_t* base, int64_t sb, int64_t st, int64_t sh, int row) -> const bf16_t* {
        const int64_t f = row < valid ? tok0 + row : 0;
        return base + (f / p.T_rows) * sb + (f % p.T_rows) * st + (int64_t)h * sh;
    };
    bf16x8 zero8;
#pragma unroll
    for (int e = 0; e < 8; e++) zero8[e] = (bf16_t)0.f;
    const int64_t mir0 = (int64_t)(p.NC - 1 - ci) * 2 * C;  // first token of chunk A in the mirror problem

    // ---- gamma (prefix sum of g inside the chunk) and beta: wave 0 ----
    if (wave == 0) {
        const int64_t at = (lane < valid ? tok0 + lane : 0) * p.H + h;
        float x = (p.g == nullptr || lane >= valid) ? 0.f : p.g[at];
#pragma unroll
        for (int off = 1; off < WAVE; off <<= 1) {
            const float y = __shfl_up(x, off, WAVE);
            if (lane >= off) x += y;
        }
        const float gl = __shfl(x, WAVE - 1, WAVE);
        const float b = lane < valid ? load_beta(p.beta, p.beta_dtype, at) : 0.f;
        s_gam[lane] = x, s_beta[lane] = b, s_e[lane] = __expf(x), s_tail[lane] = __expf(gl - x);
        p.gam[chunk * C + lane] = x;
        p.bc[chunk * C + lane] = b;
    }

    // ---- rows of q, k, v, dO: 16-byte pieces, 16 lanes per row ----
    const int p8 = t % 16;
    if (valid == 0) {
        // A chunk slot past the end of its sequence (batches laid out with the chunk count of their longest sequence):
        // what the code below would arrive at from rows of zeros - zero rows of the mirror problem, T = I, the constant
        // inverse norms - written directly; only the records are then formed as for any other chunk.
        const float r0 = p.l2norm ? rsqrtf(L2NORM_EPS) : 1.f;
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int row = t / 16 + 16 * it;
            if (p8 == 0) {
                s_rq[row] = r0, s_rk[row] = r0;
                p.rq[chunk * C + row] = r0, p.rk[chunk * C + row] = r0;
            }
            const int64_t tokA = ((int64_t)n * TM + mir0 + (C - 1 - row)) * p.H + h, tokB = tokA + (int64_t)C * p.H;
            *reinterpret_cast<bf16x8*>(p.k_m + tokA * K + 8 * p8) = zero8;
            *reinterpret_cast<bf16x8*>(p.k_m + tokB * K + 8 * p8) = zero8;
#pragma unroll
            for (int hv = 0; hv < V / 128; hv++) {
                *reinterpret_cast<bf16x8*>(p.v_m + tokA * V + 128 * hv + 8 * p8) = zero8;
                *reinterpret_cast<bf16x8*>(p.v_m + tokB * V + 128 * hv + 8 * p8) = zero8;
            }
        }
        for (int i = t; i < C * C; i += BWD_THREADS) sA[(i / C) * LDA + i % C] = (i / C == i % C) ? 1.f : 0.f;
        __syncthreads();
    } else {
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int row = t / 16 + 16 * it;
            const bool live = row < valid;
            bf16x8 qr = *reinterpret_cast<const bf16x8*>(row_of(p.q, p.q_stride_b, p.q_stride_t, p.q_stride_h, row) + 8 * p8);
            bf16x8 kr = *reinterpret_cast<const bf16x8*>(row_of(p.k, p.k_stride_b, p.k_stride_t, p.k_stride_h, row) + 8 * p8);
            if (!live) qr = zero8, kr = zero8;
            float ssq = 0.f, ssk = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) ssq += (float)qr[e] * (float)qr[e], ssk += (float)kr[e] * (float)kr[e];
#pragma unroll
            for (int off = 8; off >= 1; off >>= 1) ssq += __shfl_xor(ssq, off, WAVE), ssk += __shfl_xor(ssk, off, WAVE);
            const float rq = p.l2norm ? rsqrtf(ssq + L2NORM_EPS) : 1.f, rk = p.l2norm ? rsqrtf(ssk + L2NORM_EPS) : 1.f;
            if (p8 == 0) {
                s_rq[row] = rq, s_rk[row] = rk;
                p.rq[chunk * C + row] = rq, p.rk[chunk * C + row] = rk;
            }
            bf16x8 qb, kb;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                qb[e] = (bf16_t)((float)qr[e] * rq * p.scale);
                kb[e] = (bf16_t)((float)kr[e] * rk);
            }
            *reinterpret_cast<bf16x8*>(sQ + row * LDR + 8 * p8) = qb;
            *reinterpret_cast<bf16x8*>(sK + row * LDR + 8 * p8) = kb;
            // mirror rows: token `row` of this chunk is token 63 - row of chunks A and B
            const int64_t tokA = ((int64_t)n * TM + mir0 + (C - 1 - row)) * p.H + h, tokB = tokA + (int64_t)C * p.H;
            *reinterpret_cast<bf16x8*>(p.k_m + tokA * K + 8 * p8) = kr;
            *reinterpret_cast<bf16x8*>(p.k_m + tokB * K + 8 * p8) = qr;
#pragma unroll
            for (int hv = 0; hv < V / 128; hv++) {
                bf16x8 dr = *reinterpret_cast<const bf16x8*>(row_of(p.dout, p.d_stride_b, p.d_stride_t, p.d_stride_h, row) + 128 * hv + 8 * p8);
                if (!live) dr = zero8;
#pragma unroll
                for (int e = 0; e < 8; e++) sDOT[(128 * hv + 8 * p8 + e) * LDS64 + row] = dr[e];
                *reinterpret_cast<bf16x8*>(p.v_m + tokB * V + 128 * hv + 8 * p8) = dr;
            }
        }
        __syncthreads();

        f32x16 zero;
#pragma unroll
        for (int r = 0; r < 16; r++) zero[r] = 0.f;

        // ---- A = stril(beta_i E . K K^T) and P^T = tril(E . Q K^T)^T: wave -> tile (ti, tj) ----
        {
            const int ti = wave / 2, tj = wave % 2;
            const f32x16 KK = mma_nt(sK + 32 * ti * LDR, LDR, sK + 32 * tj * LDR, LDR, K, zero, l32, lh);
            const f32x16 QK = mma_nt(sQ + 32 * ti * LDR, LDR, sK + 32 * tj * LDR, LDR, K, zero, l32, lh);
            const int j = 32 * tj + l32;
            const float gj = s_gam[j];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int i = 32 * ti + 8 * (r / 4) + 4 * lh + r % 4;
                const float E = i >= j ? __expf(s_gam[i] - gj) : 0.f;
                sA[i * LDA + j] = i > j ? s_beta[i] * E * KK[r] : 0.f;
                sPT[j * LDS64 + i] = (bf16_t)(E * QK[r]);
            }
        }
        __syncthreads();

        // ---- P^T dO -> rows of v_m for chunk A: rows j = 32 tj + .., columns v = 32 tv + l32, tv = wave, wave + 4, .. ----
#pragma unroll
        for (int tv = wave; tv < V / 32; tv += BWD_THREADS / WAVE)
#pragma unroll
            for (int tj = 0; tj < 2; tj++) {
                const f32x16 u = mma_nt(sPT + 32 * tj * LDS64, LDS64, sDOT + 32 * tv * LDS64, LDS64, C, zero, l32, lh);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int j = 32 * tj + 8 * (r / 4) + 4 * lh + r % 4;
                    p.v_m[(((int64_t)n * TM + mir0 + (C - 1 - j)) * p.H + h) * V + 32 * tv + l32] = (bf16_t)u[r];
                }
            }

        // ---- T = (I + A)^-1 in place of A (the rows of q and k in LDS are dead: their place is the scratch) ----
        static_assert(INVERSE_SCRATCH_FLOATS * 4 <= C * LDR * 2, "the scratch of the inverse fits the rows of q");
        invert_unit_lower_64<LDA>(sA, reinterpret_cast<float*>(sQ), wave, lane);

    }

    // ---- the two records ----
    uint8_t* recA = p.rec + ((int64_t)h * ((int64_t)p.N * 2 * p.NC) + (int64_t)n * 2 * p.NC + 2 * (p.NC - 1 - ci)) * p.rec_bytes;
    uint8_t* recB = recA + p.rec_bytes;
    for (int fl = t; fl < 6 * WAVE; fl += BWD_THREADS) {
        const int f = fl / WAVE, L = fl % WAVE;
        // fragment f, lane L, element e -> entry (row, col) of the lower-triangular 64 x 64 matrix.  32x32x16 order:
        // fragments (row tile, 16-column slab) = (0,0) (0,1) (1,0) (1,1) (1,2) (1,3); a lane holds columns 4 h + 0..3 and
        // 8 + 4 h + 0..3 of the slab.  16x16x32 order: (16-row tile, 32-column slab) = (0,0) (1,0) (2,0) (2,1) (3,0) (3,1);
        // a lane holds columns 4 g + 0..3 and 16 + 4 g + 0..3 of the slab.
        const int row = p.rec16 ? 16 * (f < 2 ? f : 2 + (f - 2) / 2) + L % 16 : 32 * (f < 2 ? 0 : 1) + L % 32;
        const int col0 = p.rec16 ? 32 * (f < 2 ? 0 : f % 2) + 4 * (L / 16) : 16 * (f < 2 ? f : f - 2) + 4 * (L / 32);
        const int second = p.rec16 ? 12 : 4;  // elements 4..7 lie this many columns past e
        bf16x8 tm, id, zz;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int col = col0 + (e < 4 ? e : e + second);
            // mirrored transpose: entry (row, col) is T[63 - col][63 - row], zero above the diagonal
            tm[e] = (bf16_t)(row >= col ? sA[(C - 1 - col) * LDA + (C - 1 - row)] : 0.f);
            id[e] = (bf16_t)(row == col ? 1.f : 0.f);
            zz[e] = (bf16_t)0.f;
        }
        reinterpret_cast<bf16x8*>(recA)[fl] = tm;
        reinterpret_cast<bf16x8*>(recA + p.off_p)[fl] = id;
        reinterpret_cast<bf16x8*>(recB)[fl] = id;
        reinterpret_cast<bf16x8*>(recB + p.off_p)[fl] = zz;
    }
    if (t < C) {
        const int src = C - 1 - t;
        reinterpret_cast<float*>(recA + p.off_qs)[t] = 0.f;
        reinterpret_cast<float*>(recA + p.off_ks)[t] = -(s_beta[src] * s_e[src] * s_rk[src]);
        reinterpret_cast<float*>(recA + p.off_cs)[t] = -(s_tail[src] * s_rk[src]);
        reinterpret_cast<float*>(recB + p.off_qs)[t] = 0.f;
        reinterpret_cast<float*>(recB + p.off_ks)[t] = s_e[src] * s_rq[src] * p.scale;
        reinterpret_cast<float*>(recB + p.off_cs)[t] = 0.f;
        if (t == 0) {
            *reinterpret_cast<float*>(recA + p.off_eg) = s_e[C - 1];
            *reinterpret_cast<float*>(recB + p.off_eg) = 1.f;
        }
    }
}

}  // namespace

int launch_chunk_bwd_local(const gdn_chunk_local_args& a, hipStream_t stream) {
    ChunkLocalParams p;
    p.qs = a.qs, p.kn = a.kn, p.v = a.v, p.dout = a.dout, p.y = a.y, p.vnew = a.v_new;
    p.s0 = a.states, p.ds1 = a.dstates, p.gam = a.gamma, p.beta = a.beta;
    p.rq = a.rq, p.rk = a.rk, p.scale = a.scale;
    p.dq = a.dq, p.dk = a.dk, p.dbeta = a.dbeta, p.dgam = a.dgamma;
    p.y_mirror = static_cast<const bf16_t*>(a.y_mirror);
    p.dq_out = static_cast<bf16_t*>(a.dq_out), p.dk_out = static_cast<bf16_t*>(a.dk_out), p.dv_out = static_cast<bf16_t*>(a.dv_out);
    p.dg_out = a.dg_out, p.dbeta_out = a.dbeta_out;
    p.H = a.H, p.NC = a.NC;
    p.q_raw = static_cast<const bf16_t*>(a.q_raw), p.k_raw = static_cast<const bf16_t*>(a.k_raw);
    p.v_raw = static_cast<const bf16_t*>(a.v_raw), p.d_raw = static_cast<const bf16_t*>(a.dout_raw);
    p.q_stride_b = a.q_stride_b, p.q_stride_t = a.q_stride_t, p.q_stride_h = a.q_stride_h;
    p.k_stride_b = a.k_stride_b, p.k_stride_t = a.k_stride_t, p.k_stride_h = a.k_stride_h;
    p.v_stride_b = a.v_stride_b, p.v_stride_t = a.v_stride_t, p.v_stride_h = a.v_stride_h;
    p.d_stride_b = a.dout_stride_b, p.d_stride_t = a.dout_stride_t, p.d_stride_h = a.dout_stride_h;
    p.seq_start = a.seq_start, p.seq_len = a.seq_len, p.T_rows = a.seq_start != nullptr ? a.T_rows : a.NC * C;
    if (a.V == 512) hipLaunchKernelGGL(chunk_local_grads_kernel<512>, dim3((unsigned)a.chunks), dim3(BWD_THREADS), 0, stream, p);
    else if (a.V == 256) hipLaunchKernelGGL(chunk_local_grads_kernel<256>, dim3((unsigned)a.chunks), dim3(BWD_THREADS), 0, stream, p);
    else hipLaunchKernelGGL(chunk_local_grads_kernel<128>, dim3((unsigned)a.chunks), dim3(BWD_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}

bool chunk_bwd_local_supported(const gdn_chunk_local_args& a) { return a.K == BWD_K && (a.V == 128 || a.V == 256 || a.V == 512); }

bool chunk_bwd_prepare_supported(const gdn_chunk_bwd_prepare_args& a) {
    if (a.K != BWD_K || (a.V != 128 && a.V != 256 && a.V != 512) || a.T <= 0) return false;
    return a.seq_start != nullptr ? (a.seq_len != nullptr && a.NC > 0) : a.T % C == 0;
}

uint64_t chunk_bwd_record_bytes(const gdn_chunk_bwd_prepare_args& a) {
    const uint64_t nc = a.seq_start != nullptr ? a.NC : a.T / C;
    return (uint64_t)a.H * a.N * 2 * nc * record_layout(a.K, a.V).bytes;
}

int launch_chunk_bwd_prepare(const gdn_chunk_bwd_prepare_args& a, hipStream_t stream) {
    const RecordLayout r = record_layout(a.K, a.V);
    BwdPrepareParams p;
    p.q = static_cast<const bf16_t*>(a.q), p.k = static_cast<const bf16_t*>(a.k);
    p.dout = static_cast<const bf16_t*>(a.dout);
    p.g = a.g, p.beta = a.beta, p.beta_dtype = a.beta_dtype;
    p.q_stride_b = a.q_stride_b, p.q_stride_t = a.q_stride_t, p.q_stride_h = a.q_stride_h;
    p.k_stride_b = a.k_stride_b, p.k_stride_t = a.k_stride_t, p.k_stride_h = a.k_stride_h;
    p.d_stride_b = a.dout_stride_b, p.d_stride_t = a.dout_stride_t, p.d_stride_h = a.dout_stride_h;
    p.N = a.N, p.H = a.H, p.NC = a.seq_start != nullptr ? a.NC : a.T / C;
    p.seq_start = a.seq_start, p.seq_len = a.seq_len, p.T_rows = a.T;
    p.l2norm = (a.flags & GDN_FLAG_L2NORM) ? 1 : 0;
    p.rec16 = (a.flags & GDN_FLAG_RECORDS_16X16) ? 1 : 0;
    p.scale = a.scale;
    p.gam = a.gamma, p.bc = a.beta_packed;
    p.rq = a.rq, p.rk = a.rk;
    p.k_m = static_cast<bf16_t*>(a.k_mirror), p.v_m = static_cast<bf16_t*>(a.v_mirror);
    p.rec = static_cast<uint8_t*>(a.records);
    p.rec_bytes = r.bytes, p.off_p = r.off_p, p.off_qs = r.off_qs, p.off_ks = r.off_ks, p.off_cs = r.off_cs, p.off_eg = r.off_eg;
    const int64_t chunks = (int64_t)a.N * a.H * p.NC;
    if (a.V == 512) hipLaunchKernelGGL(chunk_bwd_prepare_kernel<512>, dim3((unsigned)chunks), dim3(BWD_THREADS), 0, stream, p);
    else if (a.V == 256) hipLaunchKernelGGL(chunk_bwd_prepare_kernel<256>, dim3((unsigned)chunks), dim3(BWD_THREADS), 0, stream, p);
    else hipLaunchKernelGGL(chunk_bwd_prepare_kernel<128>, dim3((unsigned)chunks), dim3(BWD_THREADS), 0, stream, p);
    return (int)hipGetLastError();
}

}  // namespace gdn
