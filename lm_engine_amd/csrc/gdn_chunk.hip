// Chunked forward of the gated delta rule for gfx950 (bf16 MFMA, fp32 state), chunk C = 64.
//
// Replaces fla.ops.gated_delta_rule.chunk_gated_delta_rule as called at
// lm_engine/modeling_utils/sequence_mixer_blocks/gated_deltanet/module.py:197-209.
//
// Per chunk, with gamma = cumsum(g) inside the chunk, k^ / q^ the (optionally normalised) rows
// and S0 the state at chunk start:
//
//     A_ij = beta_i e^{gamma_i - gamma_j} (k^_i . k^_j)  (i > j)        T = (I + A)^-1
//     W = T diag(beta e^gamma) K^      U = T diag(beta) V
//     V~ = U - W S0
//     O  = diag(e^gamma scale) Q^ S0 + P V~,   P_ij = scale e^{gamma_i - gamma_j} (q^_i . k^_j)  (i >= j)
//     S_C = e^{gamma_C} S0 + K~^T V~,          K~_j = e^{gamma_C - gamma_j} k^_j
//
// Two kernels:
//
//   prepare (parallel over every chunk and head): everything that does not depend on the
//       state - K K^T, the triangular inverse T, W, U, P, and the row-scaled Q~ / K~ - written
//       to a workspace record per (head, chunk) as bf16 MFMA operand fragments, i.e. in exactly
//       the register order the scan kernel consumes them (one coalesced 16 B load per lane).
//
//   scan (serial over the chunks of a sequence, parallel over sequences, heads and 16-column
//       slices of V): one wavefront owns a K x 16 slice of the fp32 state as MFMA accumulators.
//       Columns of the state evolve independently, so a wave never exchanges data with another.
//       The accumulator layout of the 16x16 MFMA (lane = column, 4 consecutive rows per register
//       quad) is fed back as the B operand of the next MFMA by fixing the order of the reduction
//       index accordingly (the fragments written by `prepare` use the same order), so neither the
//       state nor V~ ever round-trips through LDS.
//
// MFMA operand layouts used below (wave64, l = lane):
//   v_mfma_f32_16x16x32_bf16:  A[i = l%16][k = 8 (l/16) + 0..7]   B[k = 8 (l/16) + 0..7][j = l%16]
//                              D[i = 4 (l/16) + 0..3][j = l%16]
//   v_mfma_f32_16x16x4_f32:    A[i = l%16][k = l/16]   B[k = l/16][j = l%16]   D as above
//
// "Permuted reduction order": when a D tile pair (rows 32 s .. 32 s + 31 of some matrix X, held as
// two 16-row tiles) is reused as a B operand, lane (j, kq = l/16) supplies, as its 8 reduction
// entries, rows 32 s + 4 kq + 0..3 followed by rows 32 s + 16 + 4 kq + 0..3.  The matching A
// operand fragment of a row-major matrix Y therefore holds Y[m][32 s + 4 kq + 0..3] and
// Y[m][32 s + 16 + 4 kq + 0..3].

#include <type_traits>

#include "gdn_chunk_common.h"
#include "gdn_launch.h"

namespace gdn {

static int chunk_slots(const gdn_args& a) {
    const int nt = (a.T + C - 1) / C;
    const bool packed = a.cu_seqlens != nullptr && !(a.flags & GDN_FLAG_LEFT_PADDED);
    return packed ? a.T / C + a.N : a.B * nt;
}

static uint64_t chunk_off_bytes(const gdn_args& a) { return (((uint64_t)a.N + 1) * 4 + 255u) & ~(uint64_t)255u; }

bool chunk_shape_supported(const gdn_args& a) {
    if (a.dtype != GDN_BF16) return false;
    if (a.chunk != 0 && a.chunk != C) return false;
    if (a.K != 64 && a.K != 128 && a.K != 256) return false;
    if (a.V <= 0 || a.V % 32 != 0) return false;
    if (a.B <= 0 || a.T <= 0 || a.H <= 0 || a.N <= 0) return false;
    return true;
}

uint64_t chunk_record_bytes(const gdn_args& a) {
    return (uint64_t)a.H * chunk_slots(a) * record_layout(a.K, a.V).bytes;
}

// one int32 flag per record (used when prepare and scan run in one launch)
static uint64_t chunk_flag_bytes(const gdn_args& a) { return ((uint64_t)a.H * chunk_slots(a) * 4 + 255u) & ~(uint64_t)255u; }

uint64_t chunk_workspace_bytes(const gdn_args& a) {
    const RecordLayout r = record_layout(a.K, a.V);
    return chunk_off_bytes(a) + chunk_flag_bytes(a) + (uint64_t)a.H * chunk_slots(a) * r.bytes;
}

// ------------------------------------------------------------------------------------------
// chunk offsets of packed sequences: chunk_off[n] = sum_{m < n} ceil(len_m / C)
// ------------------------------------------------------------------------------------------
// Lengths are taken through packed_bounds, and the running total is capped at the number of record slots
// the workspace holds (`slots`): whatever cu_seqlens contains, no chunk gets a slot outside the workspace
// (sequences past the cap get none; a well-formed prefix never reaches it).
__global__ __launch_bounds__(256) void chunk_offsets_kernel(const int32_t* __restrict__ cu, int32_t* __restrict__ off,
                                                            int N, int total, int slots) {
    __shared__ int s_part[256];
    const int tid = threadIdx.x;
    const int per = (N + 255) / 256;
    const int begin = min(tid * per, N), end = min(begin + per, N);
    auto chunks_of = [&](int n) {
        int t0, len;
        packed_bounds(cu, n, total, t0, len);
        return (len + C - 1) / C;
    };
    int sum = 0;
    for (int n = begin; n < end; n++) sum = min(sum + chunks_of(n), slots);
    s_part[tid] = sum;
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int i = 0; i < 256; i++) {
            const int x = s_part[i];
            s_part[i] = run;
            run = min(run + x, slots);
        }
        off[N] = run;
    }
    __syncthreads();
    int run = s_part[tid];
    for (int n = begin; n < end; n++) {
        off[n] = run;
        run = min(run + chunks_of(n), slots);
    }
}

// ------------------------------------------------------------------------------------------
// prepare
// ------------------------------------------------------------------------------------------
template <int K>
__global__ __launch_bounds__(PREP_THREADS) void chunk_prepare_kernel(const ChunkParams p) {
    constexpr int LDK = K + 8;   // bf16 elements per LDS row of K / Q (16 B pad)
    constexpr int VP = 128;      // columns of V staged per pass
    constexpr int LDV = VP + 8;
    constexpr int LDA = C + 4;   // fp32 elements per LDS row of A / T
    constexpr int LDM = 20;      // fp32 elements per row of a 16 x 16 merge scratch
    constexpr int KS = K / 32;   // 32-wide reduction slabs over the key dim
    constexpr int QT_BYTES = (C * LDK * 2 > C * LDA * 4) ? C * LDK * 2 : C * LDA * 4;

    __shared__ __attribute__((aligned(16))) bf16_t sK[C * LDK];
    __shared__ __attribute__((aligned(16))) uint8_t sQT[QT_BYTES];  // Q (bf16), then T (fp32) once Q is consumed
    __shared__ __attribute__((aligned(16))) bf16_t sV[C * LDV];
    __shared__ __attribute__((aligned(16))) float sA[C * LDA];
    __shared__ __attribute__((aligned(16))) float sM[4 * 16 * LDM];
    __shared__ __attribute__((aligned(16))) float s_gam[C], s_beta[C], s_rk[C], s_rq[C], s_cw[C], s_ks[C], s_qs[C];
    bf16_t* const sQ = reinterpret_cast<bf16_t*>(sQT);
    float* const sT = reinterpret_cast<float*>(sQT);

    const int tid = threadIdx.x;
    const int lane = tid % WAVE;
    const int wave = tid / WAVE;
    const int l16 = lane % 16;  // row / column inside a 16 x 16 tile
    const int lq = lane / 16;   // which quarter of the reduction slab / which 4 rows of a D tile
    const int h = blockIdx.y;
    const int slot = blockIdx.x;

    const ChunkCoord cc = locate_chunk(p, slot);
    if (cc.len <= 0) return;
    const int len = cc.len;

    uint8_t* const rec = p.rec + ((int64_t)h * p.TC + slot) * p.rec_bytes;

    // ---- stage K, Q (and the first V pass) in LDS; rows past `len` are zero ----
    const bf16_t* kg = p.k + cc.b * p.k_stride_b + cc.t0 * p.k_stride_t + (int64_t)h * p.k_stride_h;
    const bf16_t* qg = p.q + cc.b * p.q_stride_b + cc.t0 * p.q_stride_t + (int64_t)h * p.q_stride_h;
    const bf16_t* vg = p.v + cc.b * p.v_stride_b + cc.t0 * p.v_stride_t + (int64_t)h * p.v_stride_h;
    {
        constexpr int CPR = K / 8;  // 16 B pieces per row
        constexpr int ROWS_PER_PASS = PREP_THREADS / CPR;
        const int piece = tid % CPR;
        float ssk[C / ROWS_PER_PASS], ssq[C / ROWS_PER_PASS];
#pragma unroll
        for (int it = 0; it < C / ROWS_PER_PASS; it++) {
            const int row = tid / CPR + it * ROWS_PER_PASS;
            bf16x8 kx = {}, qx = {};
            if (row < len) {
                kx = *reinterpret_cast<const bf16x8*>(kg + row * p.k_stride_t + piece * 8);
                qx = *reinterpret_cast<const bf16x8*>(qg + row * p.q_stride_t + piece * 8);
            }
            *reinterpret_cast<bf16x8*>(&sK[row * LDK + piece * 8]) = kx;
            *reinterpret_cast<bf16x8*>(&sQ[row * LDK + piece * 8]) = qx;
            float a = 0.f, b = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                a += (float)kx[e] * (float)kx[e];
                b += (float)qx[e] * (float)qx[e];
            }
            ssk[it] = a, ssq[it] = b;
        }
        if (p.l2norm) {
#pragma unroll
            for (int it = 0; it < C / ROWS_PER_PASS; it++) {
                const int row = tid / CPR + it * ROWS_PER_PASS;
                float a = ssk[it], b = ssq[it];
#pragma unroll
                for (int off = 1; off < CPR; off <<= 1) {
                    a += __shfl_xor(a, off, WAVE);
                    b += __shfl_xor(b, off, WAVE);
                }
                if (piece == 0) {
                    s_rk[row] = rsqrtf(a + L2NORM_EPS);
                    s_rq[row] = rsqrtf(b + L2NORM_EPS);
                }
            }
        } else if (tid < C) {
            s_rk[tid] = 1.f;
            s_rq[tid] = 1.f;
        }
    }

    // ---- per-token scalars: gamma = cumsum(g), beta; pad tokens get g = 0, beta = 0 ----
    if (wave == 0) {
        const int64_t sidx = (cc.b * p.T + cc.t0 + lane) * p.H + h;
        float gv = 0.f, bv = 0.f;
        if (lane < len) {
            gv = (p.g != nullptr) ? p.g[sidx] : 0.f;
            bv = load_beta(p.beta, p.beta_dtype, sidx);
        }
#pragma unroll
        for (int off = 1; off < WAVE; off <<= 1) {
            const float up = __shfl_up(gv, off, WAVE);
            if (lane >= off) gv += up;
        }
        s_gam[lane] = gv;
        s_beta[lane] = bv;
    }
    __syncthreads();
    if (tid < C) {
        const float gam = s_gam[tid], gl = s_gam[C - 1];
        s_cw[tid] = s_beta[tid] * __expf(gam) * s_rk[tid];   // column scale of T for W
        s_ks[tid] = __expf(gl - gam) * s_rk[tid];           // row scale of K~
        s_qs[tid] = __expf(gam) * p.scale * s_rq[tid];      // row scale of Q~
        if (tid == 0) *reinterpret_cast<float*>(rec + p.off_eg) = __expf(gl);
    }
    __syncthreads();

    // ---- A = strict-lower(beta_i e^{gamma_i - gamma_j} k^_i . k^_j) -> sA;  P -> record ----
    {
        const int ti = wave;  // this wave's 16 rows (of A) / 16 columns (of P^T)
        bf16x8 ka[KS], qb[KS];
#pragma unroll
        for (int s = 0; s < KS; s++) {
            ka[s] = *reinterpret_cast<const bf16x8*>(&sK[(16 * ti + l16) * LDK + 32 * s + 8 * lq]);
            qb[s] = *reinterpret_cast<const bf16x8*>(&sQ[(16 * ti + l16) * LDK + 32 * s + 8 * lq]);
        }
        f32x4 pt[4];  // P^T tiles: rows j (tile tj), column i = 16 ti + l16
#pragma unroll
        for (int tj = 0; tj < 4; tj++) {
            pt[tj] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (tj <= ti) {
                f32x4 gacc = {0.f, 0.f, 0.f, 0.f}, pacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < KS; s++) {
                    const bf16x8 kb = *reinterpret_cast<const bf16x8*>(&sK[(16 * tj + l16) * LDK + 32 * s + 8 * lq]);
                    gacc = mfma_bf16(ka[s], kb, gacc);  // D[i][j] = k_i . k_j   rows i (tile ti), col j
                    pacc = mfma_bf16(kb, qb[s], pacc);  // D[j][i] = k_j . q_i   rows j (tile tj), col i
                }
                // A tile: lane holds rows i = 16 ti + 4 lq + e, column j = 16 tj + l16
                {
                    const int j = 16 * tj + l16;
                    const float gj = s_gam[j], rkj = s_rk[j];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int i = 16 * ti + 4 * lq + e;
                        const float val = s_beta[i] * s_rk[i] * rkj * __expf(s_gam[i] - gj) * gacc[e];
                        sA[i * LDA + j] = (i > j) ? val : 0.f;
                    }
                }
                // P^T tile: lane holds rows j = 16 tj + 4 lq + e, column i = 16 ti + l16
                {
                    const int i = 16 * ti + l16;
                    const float gi = s_gam[i], qi = p.scale * s_rq[i];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int j = 16 * tj + 4 * lq + e;
                        const float val = qi * s_rk[j] * __expf(gi - s_gam[j]) * pacc[e];
                        pt[tj][e] = (i >= j) ? val : 0.f;
                    }
                }
            }
        }
        // P fragments (row tile ti, token slab s): P[i][32 s + 4 lq + e], P[i][32 s + 16 + 4 lq + e]
        bf16x8* pf = reinterpret_cast<bf16x8*>(rec + p.off_p);
        pf[(ti * 2 + 0) * WAVE + lane] = pack8(pt[0], pt[1]);
        pf[(ti * 2 + 1) * WAVE + lane] = pack8(pt[2], pt[3]);
    }

    // ---- Q~ and K~^T fragments (permuted reduction order) ----
    {
        bf16x8* qf = reinterpret_cast<bf16x8*>(rec + p.off_qs);
        for (int f = wave; f < 4 * KS; f += 4) {  // fragment (ti, s) = (f / KS, f % KS)
            const int ti = f / KS, s = f % KS;
            const int i = 16 * ti + l16;
            const float sc = s_qs[i];
            const bf16x4 a = *reinterpret_cast<const bf16x4*>(&sQ[i * LDK + 32 * s + 4 * lq]);
            const bf16x4 b = *reinterpret_cast<const bf16x4*>(&sQ[i * LDK + 32 * s + 16 + 4 * lq]);
            bf16x8 r;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                r[e] = (bf16_t)((float)a[e] * sc);
                r[4 + e] = (bf16_t)((float)b[e] * sc);
            }
            qf[f * WAVE + lane] = r;
        }
        bf16x8* kf = reinterpret_cast<bf16x8*>(rec + p.off_kt);
        for (int f = wave; f < (K / 16) * 2; f += 4) {  // fragment (td, s) = (f / 2, f % 2)
            const int td = f / 2, s = f % 2;
            const int d = 16 * td + l16;
            bf16x8 r;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int j0 = 32 * s + 4 * lq + e, j1 = j0 + 16;
                r[e] = (bf16_t)((float)sK[j0 * LDK + d] * s_ks[j0]);
                r[4 + e] = (bf16_t)((float)sK[j1 * LDK + d] * s_ks[j1]);
            }
            kf[f * WAVE + lane] = r;
        }
    }
    __syncthreads();  // A complete; Q no longer needed -> its region becomes T

    // ---- T = (I + A)^-1: forward substitution on the four 16 x 16 diagonal blocks ----
    if (wave == 0) {
        const int blk = lq, j = l16;  // lane owns column j of block `blk`
        const float* a = &sA[(16 * blk) * LDA + 16 * blk];
        float x[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float acc = (i == j) ? 1.f : 0.f;
#pragma unroll
            for (int kk = 0; kk < i; kk++) acc -= a[i * LDA + kk] * x[kk];
            x[i] = acc;
        }
#pragma unroll
        for (int i = 0; i < 16; i++) sT[(16 * blk + i) * LDA + 16 * blk + j] = x[i];
    }
    __syncthreads();

    // ---- off-diagonal blocks, three levels:  T_ij = -T_ii (sum_{k=j}^{i-1} A_ik T_kj) ----
    {
        float* const scratch = &sM[wave * 16 * LDM];
#pragma unroll
        for (int level = 1; level <= 3; level++) {
            const int bi = wave + level, bj = wave;  // block handled by this wave at this level
            const bool active = bi < 4;
            if (active) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
                for (int bk = bj; bk < bi; bk++) {
#pragma unroll
                    for (int s = 0; s < 4; s++) {
                        const float av = sA[(16 * bi + l16) * LDA + 16 * bk + 4 * s + lq];
                        const float bv = sT[(16 * bk + 4 * s + lq) * LDA + 16 * bj + l16];
                        acc = mfma_f32(av, bv, acc);
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; e++) scratch[(4 * lq + e) * LDM + l16] = acc[e];
            }
            __syncthreads();
            if (active) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < 4; s++) {
                    const float av = sT[(16 * bi + l16) * LDA + 16 * bi + 4 * s + lq];
                    const float bv = scratch[(4 * s + lq) * LDM + l16];
                    acc = mfma_f32(av, bv, acc);
                }
#pragma unroll
                for (int e = 0; e < 4; e++) sT[(16 * bi + 4 * lq + e) * LDA + 16 * bj + l16] = -acc[e];
            }
            __syncthreads();
        }
    }

    // T fragment (16 rows of tile ti, natural column order j = 32 s + 8 lq + e), columns scaled.
    auto t_frag = [&](int ti, int s, const float* colscale) -> bf16x8 {
        const int i = 16 * ti + l16;
        const int j0 = 32 * s + 8 * lq;
        const f32x4 t0 = *reinterpret_cast<const f32x4*>(&sT[i * LDA + j0]);
        const f32x4 t1 = *reinterpret_cast<const f32x4*>(&sT[i * LDA + j0 + 4]);
        const f32x4 c0 = *reinterpret_cast<const f32x4*>(&colscale[j0]);
        const f32x4 c1 = *reinterpret_cast<const f32x4*>(&colscale[j0 + 4]);
        bf16x8 r;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int ja = j0 + e, jb = j0 + 4 + e;
            r[e] = (bf16_t)(ja < i ? t0[e] * c0[e] : (ja == i ? c0[e] : 0.f));
            r[4 + e] = (bf16_t)(jb < i ? t1[e] * c1[e] : (jb == i ? c1[e] : 0.f));
        }
        return r;
    };

    // ---- W^T = K^T (T diag(cw))^T : D[d][i]; written negated as A fragments of -W ----
    {
        bf16x8* wf = reinterpret_cast<bf16x8*>(rec);
        for (int sp = wave; sp < KS; sp += 4) {  // key-dim slab: tiles td = 2 sp, 2 sp + 1
            f32x4 acc[2][4];
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int ti = 0; ti < 4; ti++) acc[a][ti] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 2; s++) {
                bf16x8 kt[2];  // A operand: K[32 s + 8 lq + e][16 td + l16]
#pragma unroll
                for (int a = 0; a < 2; a++)
#pragma unroll
                    for (int e = 0; e < 8; e++) kt[a][e] = sK[(32 * s + 8 * lq + e) * LDK + 16 * (2 * sp + a) + l16];
#pragma unroll
                for (int ti = 2 * s; ti < 4; ti++) {  // T is lower triangular: slab s only feeds rows >= 32 s
                    const bf16x8 tb = t_frag(ti, s, s_cw);
                    acc[0][ti] = mfma_bf16(kt[0], tb, acc[0][ti]);
                    acc[1][ti] = mfma_bf16(kt[1], tb, acc[1][ti]);
                }
            }
#pragma unroll
            for (int ti = 0; ti < 4; ti++) wf[(ti * KS + sp) * WAVE + lane] = pack8(-acc[0][ti], -acc[1][ti]);
        }
    }

    // ---- U = (T diag(beta)) V : D[i][n]; written as accumulator fragments [tn][lane][ti][4] ----
    {
        bf16x8 ta[4][2];
#pragma unroll
        for (int ti = 0; ti < 4; ti++)
#pragma unroll
            for (int s = 0; s < 2; s++)
                if (ti >= 2 * s) ta[ti][s] = t_frag(ti, s, s_beta);
        for (int v0 = 0; v0 < p.V; v0 += VP) {
            const int vcols = min(VP, p.V - v0);
            __syncthreads();  // previous pass of sV fully consumed
            {
                const int cpr = vcols / 8;
                for (int idx = tid; idx < C * cpr; idx += PREP_THREADS) {
                    const int row = idx / cpr, piece = idx % cpr;
                    bf16x8 x = {};
                    if (row < len) x = *reinterpret_cast<const bf16x8*>(vg + row * p.v_stride_t + v0 + piece * 8);
                    *reinterpret_cast<bf16x8*>(&sV[row * LDV + piece * 8]) = x;
                }
            }
            __syncthreads();
            for (int tl = wave; tl < vcols / 16; tl += 4) {
                f32x4 acc[4];
#pragma unroll
                for (int ti = 0; ti < 4; ti++) acc[ti] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    bf16x8 vb;  // B operand: V[32 s + 8 lq + e][16 tl + l16]
#pragma unroll
                    for (int e = 0; e < 8; e++) vb[e] = sV[(32 * s + 8 * lq + e) * LDV + 16 * tl + l16];
#pragma unroll
                    for (int ti = 2 * s; ti < 4; ti++) acc[ti] = mfma_bf16(ta[ti][s], vb, acc[ti]);
                }
                const int tn = v0 / 16 + tl;
                bf16x8* uf = reinterpret_cast<bf16x8*>(rec + p.off_u) + ((int64_t)tn * WAVE + lane) * 2;
                uf[0] = pack8(acc[0], acc[1]);
                uf[1] = pack8(acc[2], acc[3]);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// scan
// ------------------------------------------------------------------------------------------
template <int K, int NW>
__global__ __launch_bounds__(NW* WAVE) void chunk_scan_kernel(const ChunkParams p) {
    constexpr int KT = K / 16;  // 16-row tiles of the state
    constexpr int KS = K / 32;

    const int lane = threadIdx.x % WAVE;
    const int wave = threadIdx.x / WAVE;
    const int l16 = lane % 16;
    const int lq = lane / 16;

    // workgroup -> (sequence-head chain, column group); chains that share an XCD (id % 8) keep
    // all their column groups on that XCD so the record is fetched into one L2 only
    const int id = blockIdx.x;
    const int xcd = id % 8, rest = id / 8;
    const int vgroup = rest % p.scan_groups;
    const int chain = (rest / p.scan_groups) * 8 + xcd;
    if (chain >= p.N * p.H) return;
    const int tn = vgroup * NW + wave;  // 16-column tile of V owned by this wave
    if (tn * 16 >= p.V) return;
    const int n = chain / p.H, h = chain % p.H;

    int slot_begin, slot_end;
    int64_t b, seq_t0, seq_len;
    if (p.cu_seqlens == nullptr) {
        seq_len = p.pad_lens == nullptr ? p.T : min(max(p.pad_lens[n + 1] - p.pad_lens[n], 0), p.T);  // the last seq_len tokens of row n
        slot_begin = n * p.NT, slot_end = slot_begin + (int)((seq_len + C - 1) / C);
        b = n, seq_t0 = p.T - seq_len;
    } else {
        slot_begin = p.chunk_off[n], slot_end = p.chunk_off[n + 1];
        int t0, len;
        packed_bounds(p.cu_seqlens, n, p.T, t0, len);
        b = 0, seq_t0 = t0, seq_len = min(len, (slot_end - slot_begin) * C);
    }

    // state: tile t holds rows 16 t + 4 lq + e, column 16 tn + l16
    f32x4 S[KT];
    const int64_t st_off = ((int64_t)n * p.H + h) * K * p.V + (int64_t)(4 * lq) * p.V + 16 * tn + l16;
    if (p.h0 != nullptr) {
#pragma unroll
        for (int t = 0; t < KT; t++)
#pragma unroll
            for (int e = 0; e < 4; e++) S[t][e] = p.h0[st_off + (int64_t)(16 * t + e) * p.V];
    } else {
#pragma unroll
        for (int t = 0; t < KT; t++) S[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    bf16_t* const og = p.o + b * p.o_stride_b + seq_t0 * p.o_stride_t + (int64_t)h * p.o_stride_h + 16 * tn + l16;
    const uint8_t* rec = p.rec + ((int64_t)h * p.TC + slot_begin) * p.rec_bytes;

    for (int slot = slot_begin; slot < slot_end; slot++, rec += p.rec_bytes) {
        const bf16x8* wf = reinterpret_cast<const bf16x8*>(rec) + lane;
        const bf16x8* qf = reinterpret_cast<const bf16x8*>(rec + p.off_qs) + lane;
        const bf16x8* kf = reinterpret_cast<const bf16x8*>(rec + p.off_kt) + lane;
        const bf16x8* pf = reinterpret_cast<const bf16x8*>(rec + p.off_p) + lane;
        const bf16x8* uf = reinterpret_cast<const bf16x8*>(rec + p.off_u) + ((int64_t)tn * WAVE + lane) * 2;
        const float egc = *reinterpret_cast<const float*>(rec + p.off_eg);

        // state as B operand (bf16), permuted reduction order
        bf16x8 sb[KS];
#pragma unroll
        for (int s = 0; s < KS; s++) sb[s] = pack8(S[2 * s], S[2 * s + 1]);

        // V~ = U - W S0   and   O = Q~ S0
        const bf16x8 u01 = uf[0], u23 = uf[1];
        f32x4 accv[4], acco[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            accv[0][e] = (float)u01[e], accv[1][e] = (float)u01[4 + e];
            accv[2][e] = (float)u23[e], accv[3][e] = (float)u23[4 + e];
        }
#pragma unroll
        for (int ti = 0; ti < 4; ti++) {
            acco[ti] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; s++) {
                accv[ti] = mfma_bf16(wf[(ti * KS + s) * WAVE], sb[s], accv[ti]);
                acco[ti] = mfma_bf16(qf[(ti * KS + s) * WAVE], sb[s], acco[ti]);
            }
        }

        // V~ as B operand
        bf16x8 vb[2];
        vb[0] = pack8(accv[0], accv[1]);
        vb[1] = pack8(accv[2], accv[3]);

        // O += P V~
#pragma unroll
        for (int ti = 0; ti < 4; ti++)
#pragma unroll
            for (int s = 0; s < 2; s++) acco[ti] = mfma_bf16(pf[(ti * 2 + s) * WAVE], vb[s], acco[ti]);

        // S = e^{gamma_C} S + K~^T V~
#pragma unroll
        for (int t = 0; t < KT; t++) {
            f32x4 acc = S[t] * egc;
#pragma unroll
            for (int s = 0; s < 2; s++) acc = mfma_bf16(kf[(t * 2 + s) * WAVE], vb[s], acc);
            S[t] = acc;
        }

        // store O rows of this chunk (tokens past the sequence end are not written)
        const int64_t tok0 = (int64_t)(slot - slot_begin) * C;
        const int valid = (int)min((int64_t)C, seq_len - tok0);
#pragma unroll
        for (int ti = 0; ti < 4; ti++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int r = 16 * ti + 4 * lq + e;
                if (r < valid) og[(tok0 + r) * p.o_stride_t] = (bf16_t)acco[ti][e];
            }
    }

    if (p.ht != nullptr) {
#pragma unroll
        for (int t = 0; t < KT; t++)
#pragma unroll
            for (int e = 0; e < 4; e++) p.ht[st_off + (int64_t)(16 * t + e) * p.V] = S[t][e];
    }
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
int launch_chunk32(ChunkParams& p, int K, hipStream_t stream, hipEvent_t* events, int num_cus);  // gdn_chunk32.hip

static int compute_units() {
    static int cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

// K = 256: 16x16x32 kernels of this file (one workgroup per chunk in prepare, 16-column waves in the scan)
static int launch_chunk_256(ChunkParams& p, hipStream_t stream, hipEvent_t* events) {
    constexpr int K = 256;
    hipLaunchKernelGGL((chunk_prepare_kernel<K>), dim3(p.TC, p.H), dim3(PREP_THREADS), 0, stream, p);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return (int)e;
    if (events != nullptr) (void)hipEventRecord(events[2], stream);

    // waves per workgroup: as many as keep at least ~one workgroup per CU
    const int64_t chains = (int64_t)p.N * p.H;
    const int vtiles = p.V / 16;
    const int64_t waves = chains * vtiles;
    int nw = 1;
    if (waves >= 4 * 256 && vtiles % 4 == 0) nw = 4;
    else if (waves >= 2 * 256 && vtiles % 2 == 0) nw = 2;
    p.scan_groups = (vtiles + nw - 1) / nw;
    const int64_t chains8 = (chains + 7) / 8 * 8;
    const dim3 grid((unsigned)(chains8 * p.scan_groups));
    if (nw == 4) hipLaunchKernelGGL((chunk_scan_kernel<K, 4>), grid, dim3(4 * WAVE), 0, stream, p);
    else if (nw == 2) hipLaunchKernelGGL((chunk_scan_kernel<K, 2>), grid, dim3(2 * WAVE), 0, stream, p);
    else hipLaunchKernelGGL((chunk_scan_kernel<K, 1>), grid, dim3(WAVE), 0, stream, p);
    return (int)hipGetLastError();
}

int launch_chunk_fwd(const gdn_args& a, hipStream_t stream, hipEvent_t* events, const gdn_chunk_saves* saves) {
    const RecordLayout r = record_layout(a.K, a.V);
    ChunkParams p;
    p.q = static_cast<const bf16_t*>(a.q);
    p.k = static_cast<const bf16_t*>(a.k);
    p.v = static_cast<const bf16_t*>(a.v);
    p.beta = a.beta;
    p.g = a.g;
    p.h0 = a.h0;
    p.ht = a.ht;
    p.o = static_cast<bf16_t*>(a.o);
    const bool left_padded = (a.flags & GDN_FLAG_LEFT_PADDED) != 0;
    p.cu_seqlens = left_padded ? nullptr : a.cu_seqlens;
    p.pad_lens = left_padded ? a.cu_seqlens : nullptr;
    p.chunk_off = static_cast<int32_t*>(a.workspace);
    p.ready = reinterpret_cast<int32_t*>(static_cast<uint8_t*>(a.workspace) + chunk_off_bytes(a));
    p.rec = static_cast<uint8_t*>(a.workspace) + chunk_off_bytes(a) + chunk_flag_bytes(a);
    p.save_state = nullptr, p.save_vnew = nullptr, p.save_nc = 0, p.records_given = 0, p.save_every = 1, p.save_reverse = 0;
    if (saves != nullptr) {
        p.save_state = saves->states, p.save_vnew = saves->v_new, p.save_nc = saves->chunks_per_chain;
        p.save_every = saves->save_every > 0 ? saves->save_every : 1, p.save_reverse = saves->save_reverse ? 1 : 0;
        p.records_given = saves->records_given;
        if (p.records_given) p.chunk_off = nullptr, p.ready = nullptr, p.rec = static_cast<uint8_t*>(a.workspace);
    }
    p.q_stride_b = a.q_stride_b, p.q_stride_t = a.q_stride_t, p.q_stride_h = a.q_stride_h;
    p.k_stride_b = a.k_stride_b, p.k_stride_t = a.k_stride_t, p.k_stride_h = a.k_stride_h;
    p.v_stride_b = a.v_stride_b, p.v_stride_t = a.v_stride_t, p.v_stride_h = a.v_stride_h;
    p.o_stride_b = a.o_stride_b, p.o_stride_t = a.o_stride_t, p.o_stride_h = a.o_stride_h;
    p.B = a.B, p.T = a.T, p.H = a.H, p.V = a.V, p.N = a.N;
    p.NT = (a.T + C - 1) / C;
    p.TC = chunk_slots(a);
    p.beta_dtype = a.beta_dtype;
    p.l2norm = (a.flags & GDN_FLAG_L2NORM) ? 1 : 0;
    p.scale = a.scale;
    p.rec_bytes = r.bytes, p.off_qs = r.off_qs, p.off_kt = r.off_kt, p.off_ks = r.off_ks, p.off_cs = r.off_cs, p.off_p = r.off_p, p.off_u = r.off_u;
    p.off_eg = r.off_eg;
    p.scan_groups = 1;
    p.fused = (a.flags & GDN_FLAG_FUSED_LAUNCH) ? 1 : 0;

    auto mark = [&](int i) {
        if (events != nullptr) (void)hipEventRecord(events[i], stream);
    };
    mark(0);
    if (p.cu_seqlens != nullptr) {
        hipLaunchKernelGGL(chunk_offsets_kernel, dim3(1), dim3(256), 0, stream, p.cu_seqlens, p.chunk_off, p.N, p.T, p.TC);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return (int)e;
    }
    mark(1);
    const int rc = (a.K == 256) ? launch_chunk_256(p, stream, events) : launch_chunk32(p, a.K, stream, events, compute_units());
    mark(3);
    return rc;
}

}  // namespace gdn
