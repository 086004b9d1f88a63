// The gated matrix memory over prompt portions on the matrix cores (bf16 operands, fp32 sums, fp32 state).
//
// The recurrence of a head (state S [d, dv], normaliser n [d], running maximum m; see mixer_parts.hip),
//     m_t = max(lf_t + m_(t-1), li_t);  S_t = e^(lf_t + m_(t-1) - m_t) S_(t-1) + e^(li_t - m_t) k_t v_t^T;  n_t likewise,
// is unrolled over a chunk of 64 tokens. With F_t the running sum of lf inside the chunk, a_s = li_s - F_s and m_0, S_0, n_0
// what the chunk starts from:
//     m_t = F_t + max(m_0, max_(s<=t) a_s)                                   (the same numbers as token by token)
//     S_t = e^(F_t + m_0 - m_t) S_0 + sum_(s<=t) e^(a_s + F_t - m_t) k_s v_s^T
// so the read-out of all 64 tokens is two matrix products, P V with P_ts = (q_t . k_s) e^(a_s + F_t - m_t) for s <= t, and
// Q S_0 with rows weighted by e^(F_t + m_0 - m_t); n_t . q_t is the row sum of P plus the weighted n_0 . q_t; and the state
// after the chunk is e^(F_L + m_0 - m_L) S_0 + K^T diag(e^(a_s + F_L - m_L)) V, one more product. Every exponent is <= 0.
// Gates, maxima, weights, sums, the state and the norm of the read-out are fp32; P, the weighted values and a copy of
// S_0 enter the products as bf16 (as the weights of attention do).
//
// Two ways of running it. In turn: a workgroup of four waves per (head, row of the batch) walks over the row's chunks
// (MC_SEQ). In three passes, for rows of many chunks: every chunk's state as if it started from nothing, all chunks at
// once (MC_LOCAL: e^(a_s - max a) weights, its own maximum m_loc = F_L + max a); a scan over a row's chunks that turns
// those into the state every chunk starts from, m_end = max(F_L + m_start, m_loc),
// S_end = e^(F_L + m_start - m_end) S_start + e^(m_loc - m_end) S_loc, element by element in fp32 (it also advances the
// request's state); and every chunk's read-out from its start state, all chunks at once (MC_READ). The passes meet in a
// buffer of the caller's, per chunk and head S [d, dv], n [d], its own maximum, F_L and the maximum it starts from.
//
// In turn, a workgroup of four waves per (head, row of the batch) walks over the row's chunks. S^T lives in the accumulators of
// the state product for the whole walk: wave w owns the value channels [w dv / 4, (w + 1) dv / 4). Operands are staged in
// LDS in the layouts that v_mfma_f32_32x32x16_bf16 reads with one 16-byte load a lane: a row operand as [row][k], a
// column operand as [column][k].
#include "ka_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 mc_bf16x8;
typedef __attribute__((ext_vector_type(16))) float mc_floatx16;

constexpr int MC_CHUNK = 64;
constexpr int MC_THREADS = 256;
constexpr int MC_PAD = 8;                   // elements a row of an LDS tile is longer than its data: spreads rows over banks
constexpr int MC_SEQ = 0, MC_LOCAL = 1, MC_READ = 2;
constexpr int MC_SCAN_CHUNKS = 1024;        // most chunks of one row that the scan keeps the weights of in LDS

struct ChunkArgs {
    const bf16_t* q; const bf16_t* k; const bf16_t* v; const bf16_t* gate;
    long stride;
    const float* pre;              // fp32 [n, 2 heads]
    float* state;                  // fp32 [state rows, heads, d dv + d + 1]
    const int* cu_q;
    const int* row_slot;
    const float* gain;             // fp32 [heads dv] or null
    bf16_t* out;
    long out_stride;
    int heads;
    float q_scale, cap, eps;
    float* chunks;                 // the passes' buffer: fp32 [chunks, heads, d dv + d + 3]
    int n_rows;
};

// The row and the first token of chunk `g` of the batch (chunks numbered row by row); false: behind the last chunk.
__device__ __forceinline__ bool mc_find_chunk(const int* cu_q, int n_rows, int g, int& r, int& t0, int& t1, int& c0) {
    int base = 0;
    for (r = 0; r < n_rows; ++r) {
        t0 = cu_q[r];
        t1 = cu_q[r + 1];
        const int nc = (t1 - t0 + MC_CHUNK - 1) / MC_CHUNK;
        if (g < base + nc) {
            c0 = t0 + (g - base) * MC_CHUNK;
            return true;
        }
        base += nc;
    }
    return false;
}

__device__ __forceinline__ float mc_running_max(float x, int lane) {
    for (int off = 1; off < KA_WAVE; off <<= 1) {
        const float y = __shfl_up(x, off);
        if (lane >= off) x = fmaxf(x, y);
    }
    return x;
}

// ND: d = 32 ND; NJ: dv = 128 NJ. MODE: MC_SEQ (grid (heads, rows)), MC_LOCAL or MC_READ (grid (heads, chunks)).
template <int ND, int NJ, int MODE>
__global__ void __launch_bounds__(MC_THREADS) matrix_memory_chunk_kernel(ChunkArgs a) {
    constexpr int D = 32 * ND, DV = 128 * NJ, WJ = 32 * NJ;       // WJ: value channels a wave owns
    constexpr int LQ = D + MC_PAD, LC = MC_CHUNK + MC_PAD;
    extern __shared__ __attribute__((aligned(16))) unsigned char mc_lds[];
    bf16_t* Qs = reinterpret_cast<bf16_t*>(mc_lds);               // [64][LQ]
    bf16_t* Ks = Qs + MC_CHUNK * LQ;                              // [64][LQ]
    bf16_t* KTs = Ks + MC_CHUNK * LQ;                             // [D][LC]
    bf16_t* VTs = KTs + D * LC;                                   // [DV][LC]
    bf16_t* Ps = VTs + DV * LC;                                   // [64][LC]
    bf16_t* STs = Ps + MC_CHUNK * LC;                             // [DV][LQ]: the state the chunk starts from, transposed
    float* fa = reinterpret_cast<float*>(STs + DV * LQ);          // a_s = li_s - F_s
    float* fb = fa + MC_CHUNK;                                    // b_t = F_t - m_t
    float* fm = fb + MC_CHUNK;                                    // m_t
    float* fu = fm + MC_CHUNK;                                    // u_s = e^(a_s + b_L)
    float* nq = fu + MC_CHUNK;                                    // n_0 . q_t (times the scale)
    float* rowsum = nq + MC_CHUNK;                                // [2][64]: row sums of P by column block
    float* sq = rowsum + 2 * MC_CHUNK;                            // [4][64]: sums of squares of the read-out by wave
    float* nvec = sq + 4 * MC_CHUNK;                              // [D]: n
    float* nnew = nvec + D;                                       // [D]
    float* scal = nnew + D;                                       // [3]: m_0 of the next chunk, c_L, F_L

    const int head = blockIdx.x, tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / KA_WAVE), lane = tid % KA_WAVE;
    const int col = lane % 32, half = lane / 32;
    int r = blockIdx.y, t0, t1, first = 0;
    if constexpr (MODE == MC_SEQ) {
        t0 = a.cu_q[r];
        t1 = a.cu_q[r + 1];
        first = t0;
    } else {
        if (!mc_find_chunk(a.cu_q, a.n_rows, blockIdx.y, r, t0, t1, first)) return;
        t1 = min(t1, first + MC_CHUNK);                 // (this workgroup's chunk alone)
    }
    if (t0 >= t1) return;
    const int slot = a.row_slot[r];
    if (slot < 0) {
        if constexpr (MODE != MC_LOCAL)
            for (int t = first; t < t1; ++t)
                for (int j = tid; j < DV; j += MC_THREADS) a.out[(size_t)t * a.out_stride + head * DV + j] = (bf16_t)0.f;
        return;
    }
    // where the state comes from and goes to: the request's row (in turn), the chunk's record of the passes' buffer
    float* st = MODE == MC_SEQ ? a.state + ((size_t)slot * a.heads + head) * (D * DV + D + 1)
                               : a.chunks + ((size_t)blockIdx.y * a.heads + head) * (D * DV + D + 3);
    // S^T in accumulators: tile (jb, db), register i of a lane: value channel wave WJ + jb 32 + (i / 4) 8 + half 4 + i % 4,
    // key channel db 32 + col
    mc_floatx16 S[NJ][ND];
#pragma unroll
    for (int jb = 0; jb < NJ; ++jb)
#pragma unroll
        for (int db = 0; db < ND; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int j = wave * WJ + jb * 32 + (i / 4) * 8 + half * 4 + i % 4, dd = db * 32 + col;
                S[jb][db][i] = MODE == MC_SEQ ? st[(size_t)dd * DV + j] : 0.f;
            }
    for (int e = tid; e < D; e += MC_THREADS) nvec[e] = MODE == MC_LOCAL ? 0.f : st[D * DV + e];
    // (a chunk as if it started from nothing; a read-out from the maximum that the scan has left for its chunk)
    float m0 = MODE == MC_LOCAL ? -INFINITY : st[D * DV + D + (MODE == MC_READ ? 2 : 0)];

    for (int c0 = first; c0 < t1; c0 += MC_CHUNK) {
        const int valid = min(MC_CHUNK, t1 - c0);
        __syncthreads();                   // (the chunk before is done with every tile)
        // the state the chunk starts from, as a column operand
        if constexpr (MODE == MC_SEQ) {
#pragma unroll
            for (int jb = 0; jb < NJ; ++jb)
#pragma unroll
                for (int db = 0; db < ND; ++db)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int j = wave * WJ + jb * 32 + (i / 4) * 8 + half * 4 + i % 4, dd = db * 32 + col;
                        STs[j * LQ + dd] = (bf16_t)S[jb][db][i];
                    }
        } else if constexpr (MODE == MC_READ) {
            for (int e = tid; e < D * DV; e += MC_THREADS) STs[(e % DV) * LQ + e / DV] = (bf16_t)st[e];
        }
        // queries and keys as they are (rows behind the row's last token: zeros), keys and values transposed
        // (neighbouring lanes take neighbouring tokens: the transposed tiles are then written along their rows)
        for (int e = tid; e < MC_CHUNK * (D / 8); e += MC_THREADS) {
            const int t = e % MC_CHUNK, piece = e / MC_CHUNK;
            mc_bf16x8 qv, kv;
#pragma unroll
            for (int u = 0; u < 8; ++u) { qv[u] = (bf16_t)0.f; kv[u] = (bf16_t)0.f; }
            if (t < valid) {
                const size_t at = (size_t)(c0 + t) * a.stride + head * D + piece * 8;
                qv = *reinterpret_cast<const mc_bf16x8*>(a.q + at);
                kv = *reinterpret_cast<const mc_bf16x8*>(a.k + at);
            }
            *reinterpret_cast<mc_bf16x8*>(Qs + t * LQ + piece * 8) = qv;
            *reinterpret_cast<mc_bf16x8*>(Ks + t * LQ + piece * 8) = kv;
#pragma unroll
            for (int u = 0; u < 8; ++u) KTs[(piece * 8 + u) * LC + t] = kv[u];
        }
        for (int e = tid; e < MC_CHUNK * (DV / 8); e += MC_THREADS) {
            const int t = e % MC_CHUNK, piece = e / MC_CHUNK;
            mc_bf16x8 vv;
#pragma unroll
            for (int u = 0; u < 8; ++u) vv[u] = (bf16_t)0.f;
            if (t < valid) vv = *reinterpret_cast<const mc_bf16x8*>(a.v + (size_t)(c0 + t) * a.stride + head * DV + piece * 8);
#pragma unroll
            for (int u = 0; u < 8; ++u) VTs[(piece * 8 + u) * LC + t] = vv[u];
        }
        // the gates of the chunk: one wave, a token a lane
        if (wave == 0) {
            float li = -INFINITY, lf = 0.f;              // (behind the last token: no input, nothing forgotten)
            if (lane < valid) {
                const size_t at = (size_t)(c0 + lane) * 2 * a.heads;
                li = a.cap * tanhf(a.pre[at + head] / a.cap);
                const float z = a.cap * tanhf(a.pre[at + a.heads + head] / a.cap);
                lf = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
            }
            const float F = ka_wave_running_sum(lf);
            const float as = li - F;
            const float top = fmaxf(m0, mc_running_max(as, lane));
            fa[lane] = as;
            fb[lane] = -top;                             // F_t - m_t with m_t = F_t + top
            fm[lane] = F + top;
            const float b_last = -ka_lane_value(top, KA_WAVE - 1);
            fu[lane] = expf(as + b_last);
            if (lane == 0) {
                scal[0] = ka_lane_value(F + top, KA_WAVE - 1);
                scal[1] = expf(m0 + b_last);
                scal[2] = ka_lane_value(F, KA_WAVE - 1);
            }
        }
        __syncthreads();
        if constexpr (MODE != MC_LOCAL) {
        // n_0 . q_t, a token a thread
        if (tid < MC_CHUNK) {
            float acc = 0.f;
            for (int dd = 0; dd < D; ++dd) acc += nvec[dd] * (float)Qs[tid * LQ + dd];
            nq[tid] = acc * a.q_scale;
        }
        // scores of the chunk against itself: wave w computes the block of tokens tb = w / 2 against keys sb = w % 2
        {
            const int tb = wave / 2, sb = wave % 2;
            mc_floatx16 g;
#pragma unroll
            for (int i = 0; i < 16; ++i) g[i] = 0.f;
            // (rows are queries, columns keys: a lane holds 16 queries' scores against ONE key)
#pragma unroll
            for (int kk = 0; kk < D / 16; ++kk) {
                const mc_bf16x8 qa = *reinterpret_cast<const mc_bf16x8*>(Qs + (tb * 32 + col) * LQ + kk * 16 + half * 8);
                const mc_bf16x8 kb = *reinterpret_cast<const mc_bf16x8*>(Ks + (sb * 32 + col) * LQ + kk * 16 + half * 8);
                g = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa, kb, g, 0, 0, 0);
            }
            const int s = sb * 32 + col;
            const float a_s = fa[s];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int t = tb * 32 + (i / 4) * 8 + half * 4 + i % 4;
                const float p = s <= t ? g[i] * a.q_scale * expf(a_s + fb[t]) : 0.f;
                Ps[t * LC + s] = (bf16_t)p;
                const float sum = ka_lanes_reduce<1, 32>(p, KaSum{});
                if (col == 0) rowsum[sb * MC_CHUNK + t] = sum;
            }
        }
        __syncthreads();
        // read-out: O = P V + diag(e^(m_0 + b_t)) scale Q S_0, the wave's value channels of all 64 tokens
        mc_floatx16 O[2][NJ];
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int jb = 0; jb < NJ; ++jb) {
                mc_floatx16 carry;
#pragma unroll
                for (int i = 0; i < 16; ++i) carry[i] = 0.f;
#pragma unroll
                for (int kk = 0; kk < D / 16; ++kk) {
                    const mc_bf16x8 qa = *reinterpret_cast<const mc_bf16x8*>(Qs + (tb * 32 + col) * LQ + kk * 16 + half * 8);
                    const mc_bf16x8 sb = *reinterpret_cast<const mc_bf16x8*>(STs + (wave * WJ + jb * 32 + col) * LQ + kk * 16 + half * 8);
                    carry = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa, sb, carry, 0, 0, 0);
                }
                mc_floatx16 acc;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int t = tb * 32 + (i / 4) * 8 + half * 4 + i % 4;
                    acc[i] = carry[i] * a.q_scale * expf(m0 + fb[t]);
                }
#pragma unroll
                for (int kk = 0; kk < MC_CHUNK / 16; ++kk) {
                    const mc_bf16x8 pa = *reinterpret_cast<const mc_bf16x8*>(Ps + (tb * 32 + col) * LC + kk * 16 + half * 8);
                    const mc_bf16x8 vb = *reinterpret_cast<const mc_bf16x8*>(VTs + (wave * WJ + jb * 32 + col) * LC + kk * 16 + half * 8);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pa, vb, acc, 0, 0, 0);
                }
                O[tb][jb] = acc;
            }
        // divided by max(|n_t . q_t|, e^(-m_t)) + 1e-6, then this wave's share of every token's sum of squares
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int t = tb * 32 + (i / 4) * 8 + half * 4 + i % 4;
                const float dot = expf(m0 + fb[t]) * nq[t] + (rowsum[t] + rowsum[MC_CHUNK + t]);
                const float den = fmaxf(fabsf(dot), expf(-fm[t])) + 1e-6f;
                float ssq = 0.f;
#pragma unroll
                for (int jb = 0; jb < NJ; ++jb) {
                    O[tb][jb][i] /= den;
                    ssq += O[tb][jb][i] * O[tb][jb][i];
                }
                ssq = ka_lanes_reduce<1, 32>(ssq, KaSum{});
                if (col == 0) sq[wave * MC_CHUNK + t] = ssq;
            }
        __syncthreads();
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int t = tb * 32 + (i / 4) * 8 + half * 4 + i % 4;
                if (t < valid) {
                    const float total = (sq[t] + sq[MC_CHUNK + t]) + (sq[2 * MC_CHUNK + t] + sq[3 * MC_CHUNK + t]);
                    const float rr = 1.0f / sqrtf(total / (float)DV + a.eps);
#pragma unroll
                    for (int jb = 0; jb < NJ; ++jb) {
                        const int c = head * DV + wave * WJ + jb * 32 + col;
                        const size_t tok = (size_t)(c0 + t);
                        const float g = a.gate ? 1.0f / (1.0f + expf(-(float)a.gate[tok * a.stride + c])) : 1.f;
                        a.out[tok * a.out_stride + c] = (bf16_t)(O[tb][jb][i] * rr * (a.gain ? a.gain[c] : 1.f) * g);
                    }
                }
            }
        }   // (MODE != MC_LOCAL)
        if constexpr (MODE == MC_READ) return;
        // the state after the chunk: S^T <- c_L S^T + (diag(u) V)^T K, n <- c_L n + K^T u
        const float c_last = scal[1];
        if (tid < D) {
            float acc = c_last * nvec[tid];
            for (int s = 0; s < MC_CHUNK; ++s) acc += fu[s] * (float)KTs[tid * LC + s];
            nnew[tid] = acc;
        }
#pragma unroll
        for (int jb = 0; jb < NJ; ++jb) {
#pragma unroll
            for (int db = 0; db < ND; ++db)
#pragma unroll
                for (int i = 0; i < 16; ++i) S[jb][db][i] *= c_last;
#pragma unroll
            for (int kk = 0; kk < MC_CHUNK / 16; ++kk) {
                const int s0 = kk * 16 + half * 8;
                const mc_bf16x8 vraw = *reinterpret_cast<const mc_bf16x8*>(VTs + (wave * WJ + jb * 32 + col) * LC + s0);
                mc_bf16x8 va;
#pragma unroll
                for (int u = 0; u < 8; ++u) va[u] = (bf16_t)((float)vraw[u] * fu[s0 + u]);
#pragma unroll
                for (int db = 0; db < ND; ++db) {
                    const mc_bf16x8 kb = *reinterpret_cast<const mc_bf16x8*>(KTs + (db * 32 + col) * LC + s0);
                    S[jb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, kb, S[jb][db], 0, 0, 0);
                }
            }
        }
        m0 = scal[0];
        __syncthreads();
        if (tid < D) nvec[tid] = nnew[tid];
    }
    __syncthreads();
#pragma unroll
    for (int jb = 0; jb < NJ; ++jb)
#pragma unroll
        for (int db = 0; db < ND; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int j = wave * WJ + jb * 32 + (i / 4) * 8 + half * 4 + i % 4, dd = db * 32 + col;
                st[(size_t)dd * DV + j] = S[jb][db][i];
            }
    for (int e = tid; e < D; e += MC_THREADS) st[D * DV + e] = nvec[e];
    if (tid == 0) {
        st[D * DV + D] = m0;
        if constexpr (MODE == MC_LOCAL) st[D * DV + D + 1] = scal[2];
    }
}

// The scan of the three passes: workgroups per (head, row, slice of the state's numbers). Every workgroup works out the
// row's chain of maxima from the chunks' records (their own maxima and sums of log forget gates, gathered in parallel)
// and with it, per chunk, the two weights of its step; every thread then carries its few numbers of S and n through the
// chunks, writing into each chunk's record the state it starts from, and the request's state at the end. The slice 0
// workgroup also leaves every chunk the maximum it starts from, and the request's at the end.
constexpr int MC_SCAN_PER_THREAD = 4;
__global__ void __launch_bounds__(MC_THREADS) matrix_memory_scan_kernel(ChunkArgs a, int D, int DV) {
    __shared__ float w_old[MC_SCAN_CHUNKS], w_new[MC_SCAN_CHUNKS], m_start[MC_SCAN_CHUNKS];
    const int head = blockIdx.x, r = blockIdx.y, tid = threadIdx.x;
    const int t0 = a.cu_q[r], t1 = a.cu_q[r + 1];
    if (t0 >= t1) return;
    const int slot = a.row_slot[r];
    if (slot < 0) return;
    int base = 0;
    for (int q = 0; q < r; ++q) base += (a.cu_q[q + 1] - a.cu_q[q] + MC_CHUNK - 1) / MC_CHUNK;
    const int nc = (t1 - t0 + MC_CHUNK - 1) / MC_CHUNK;
    const int per = D * DV + D;
    float* st = a.state + ((size_t)slot * a.heads + head) * (per + 1);
    float* rec = a.chunks + ((size_t)base * a.heads + head) * (per + 3);
    const size_t step = (size_t)a.heads * (per + 3);
    for (int c = tid; c < nc; c += MC_THREADS) {
        w_old[c] = rec[c * step + per + 1];         // (for now: the chunk's sum of log forget gates, and its own maximum)
        w_new[c] = rec[c * step + per];
    }
    __syncthreads();
    if (tid == 0) {
        float m = st[per];
        for (int c = 0; c < nc; ++c) {
            const float f_all = w_old[c], m_loc = w_new[c];
            const float m_end = fmaxf(f_all + m, m_loc);
            w_old[c] = expf(f_all + m - m_end);
            w_new[c] = expf(m_loc - m_end);
            m_start[c] = m;
            m = m_end;
        }
        if (blockIdx.z == 0) st[per] = m;
    }
    __syncthreads();
    if (blockIdx.z == 0)
        for (int c = tid; c < nc; c += MC_THREADS) rec[c * step + per + 2] = m_start[c];
    const int lo = blockIdx.z * MC_THREADS * MC_SCAN_PER_THREAD;
    for (int e = lo + tid; e < min(per, lo + MC_THREADS * MC_SCAN_PER_THREAD); e += MC_THREADS) {
        float cur = st[e];
        int c = 0;
        for (; c + 3 < nc; c += 4) {        // (four records in flight)
            float x[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) x[u] = rec[(c + u) * step + e];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                rec[(c + u) * step + e] = cur;
                cur = w_old[c + u] * cur + w_new[c + u] * x[u];
            }
        }
        for (; c < nc; ++c) {
            const float x = rec[c * step + e];
            rec[c * step + e] = cur;
            cur = w_old[c] * cur + w_new[c] * x;
        }
        st[e] = cur;
    }
}

template <int ND, int NJ>
static size_t mc_lds_bytes() {
    constexpr int D = 32 * ND, DV = 128 * NJ, LQ = D + MC_PAD, LC = MC_CHUNK + MC_PAD;
    return sizeof(bf16_t) * ((size_t)2 * MC_CHUNK * LQ + (size_t)D * LC + (size_t)DV * LC + (size_t)MC_CHUNK * LC + (size_t)DV * LQ)
        + sizeof(float) * (5 * MC_CHUNK + 2 * MC_CHUNK + 4 * MC_CHUNK + 2 * D + 4);
}

// Whether the kernel covers heads of these sizes: keys of 32, 64 or 128 channels, values of 128 or 256 (128 x 256: its
// tiles do not fit in LDS).
KA_API int ka_matrix_memory_chunks_supported(int d, int dv) {
    return (d == 32 || d == 64 || d == 128) && (dv == 128 || dv == 256) && !(d == 128 && dv == 256) ? 1 : 0;
}

// Floats of the passes' buffer for a step of `n` tokens in `n_rows` rows (every row may end in a part of a chunk).
KA_API long ka_matrix_memory_chunks_scratch(int n, int n_rows, int heads, int d, int dv) {
    return (long)(n / MC_CHUNK + n_rows) * heads * ((long)d * dv + d + 3);
}

// chunks != nullptr (of at least ka_matrix_memory_chunks_scratch floats; n = the step's tokens): the three passes;
// nullptr: every row's chunks in turn.
KA_API int ka_matrix_memory_chunks_bf16(const void* q, const void* k, const void* v, const void* gate, long stride,
                                        const float* pre, float* state, const int* cu_q, const int* row_slot,
                                        const float* gain, void* out, long out_stride, int n_rows, int heads, int d, int dv,
                                        float q_scale, float cap, float eps, float* chunks, int n, hipStream_t stream) {
    const char* who = "ka_matrix_memory_chunks_bf16";
    KA_CHECK(n_rows >= 0 && heads > 0 && ka_matrix_memory_chunks_supported(d, dv), "%s: heads of %d x %d not covered", who, d, dv);
    KA_CHECK(cap > 0.f && eps >= 0.f, "%s: the gates' cap must be positive", who);
    KA_CHECK(heads <= 65535 && n_rows <= 65535, "%s: too many heads or rows", who);
    KA_CHECK((uintptr_t)q % 16 == 0 && (uintptr_t)k % 16 == 0 && (uintptr_t)v % 16 == 0 && stride % 8 == 0,
             "%s: operands must be 16-byte aligned", who);
    if (n_rows == 0) return 0;
    const int n_chunks = n / MC_CHUNK + n_rows;
    // (a row of more chunks than the scan keeps weights for, or more chunks than a grid takes: in turn)
    if (chunks != nullptr && (n / MC_CHUNK + 1 > MC_SCAN_CHUNKS || n_chunks > 65535)) chunks = nullptr;
    ChunkArgs a{(const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, (const bf16_t*)gate, stride, pre, state, cu_q, row_slot,
                gain, (bf16_t*)out, out_stride, heads, q_scale, cap, eps, chunks, n_rows};
    const dim3 block(MC_THREADS);
    const int scan_slices = ka_cdiv((long)d * dv + d, MC_THREADS * MC_SCAN_PER_THREAD);
#define MC_LAUNCH_MODE(ND, NJ, MODE, GRID)                                                                                  \
    do {                                                                                                                    \
        static bool sized = false;                                                                                          \
        if (!sized) {                                                                                                       \
            (void)hipFuncSetAttribute((const void*)matrix_memory_chunk_kernel<ND, NJ, MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
            sized = true;                                                                                                   \
        }                                                                                                                   \
        const size_t lds = mc_lds_bytes<ND, NJ>();                                                                          \
        hipLaunchKernelGGL((matrix_memory_chunk_kernel<ND, NJ, MODE>), GRID, block, lds, stream, a);                        \
    } while (0)
#define MC_LAUNCH(ND, NJ)                                                                                                   \
    if (d == 32 * ND && dv == 128 * NJ) {                                                                                   \
        if (chunks == nullptr) {                                                                                            \
            MC_LAUNCH_MODE(ND, NJ, MC_SEQ, dim3(heads, n_rows));                                                            \
        } else {                                                                                                            \
            MC_LAUNCH_MODE(ND, NJ, MC_LOCAL, dim3(heads, n_chunks));                                                        \
            hipLaunchKernelGGL(matrix_memory_scan_kernel, dim3(heads, n_rows, scan_slices), block, 0, stream, a, d, dv);    \
            MC_LAUNCH_MODE(ND, NJ, MC_READ, dim3(heads, n_chunks));                                                         \
        }                                                                                                                   \
    }
    MC_LAUNCH(1, 1) MC_LAUNCH(2, 1) MC_LAUNCH(4, 1) MC_LAUNCH(1, 2) MC_LAUNCH(2, 2)
#undef MC_LAUNCH
#undef MC_LAUNCH_MODE
    KA_LAUNCH_CHECK();
    return 0;
}
