// Embedding gather, LayerNorm and rotary + paged cache write.
//
// The residual stream is fp32 in every precision mode; these kernels read and write
// it as fp32 and convert only at the boundary to the model's storage type.
#include "ka_common.h"

KA_API int ka_version() { return 1; }

// ----------------------------------------------------------------------------
// Embedding: out[t, :] = table[ids[t], :] as fp32. A row with ids[t] == -1 is left as it
// is (its embedding was given by the caller). ids[t] <= -2 names the entry -2 - ids[t] of
// `pending`, a device table of token ids that an earlier step's sampling filled: the id of
// a decoded token can so reach the next step without passing through the host.
// ----------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             const int* __restrict__ pending, int n_pending, int vocab,
                             float* __restrict__ out, int dim, float scale) {
    int t = blockIdx.x;
    int id = ids[t];
    if (id == -1) return;
    if (id < 0) {
        int at = -2 - id;
        if (!pending || at >= n_pending) return;
        id = pending[at];
        if ((unsigned)id >= (unsigned)vocab) id = 0;   // never an address outside the table
    }
    const T* src = table + (size_t)id * dim;
    float* dst = out + (size_t)t * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) dst[d] = ka_to_float(src[d]) * scale;
}

// `scale`: a factor on the looked-up rows (1 for none; rows with id -1, which are given from
// outside, are not touched).
KA_API int ka_embed(const void* table, int table_dtype, const int* ids, const int* pending, int n_pending,
                    int vocab, float* out, int n, int dim, float scale, hipStream_t stream) {
    KA_CHECK(n >= 0 && dim > 0 && vocab > 0 && n_pending >= 0, "ka_embed: bad sizes n=%d dim=%d vocab=%d", n, dim, vocab);
    if (n == 0) return 0;
    dim3 grid(n), block(256);
    if (table_dtype == KA_F32)
        hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, (const float*)table, ids, pending, n_pending,
                           vocab, out, dim, scale);
    else if (table_dtype == KA_BF16)
        hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)table, ids, pending,
                           n_pending, vocab, out, dim, scale);
    else
        KA_CHECK(false, "ka_embed: unsupported table dtype %d", table_dtype);
    KA_LAUNCH_CHECK();
    return 0;
}

// logits *= scale; then, with cap > 0, logits = cap * tanh(logits / cap): what some architectures do
// to their logits before sampling.
__global__ void adjust_logits_kernel(float* __restrict__ logits, long count, float scale, float cap) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float x = logits[i] * scale;
    if (cap > 0.f) x = cap * tanhf(x / cap);
    logits[i] = x;
}

KA_API int ka_adjust_logits(float* logits, long count, float scale, float cap, hipStream_t stream) {
    KA_CHECK(count >= 0 && cap >= 0.f, "ka_adjust_logits: bad count %ld or cap %g", count, cap);
    if (count == 0) return 0;
    KA_CHECK((count + 255) / 256 < (1L << 31), "ka_adjust_logits: too many values");
    hipLaunchKernelGGL(adjust_logits_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, logits, count, scale, cap);
    KA_LAUNCH_CHECK();
    return 0;
}

// out[rows[i], :] = src[i, :] (given embeddings spliced into the stream); a negative row: nothing
// (the unused end of a list of fixed length).
template <typename T>
__global__ void scatter_rows_kernel(const T* __restrict__ src, const int* __restrict__ rows,
                                    float* __restrict__ out, int dim) {
    int i = blockIdx.x;
    if (rows[i] < 0) return;
    const T* s = src + (size_t)i * dim;
    float* dst = out + (size_t)rows[i] * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) dst[d] = ka_to_float(s[d]);
}

KA_API int ka_scatter_rows(const void* src, int src_dtype, const int* rows, float* out, int m,
                           int dim, hipStream_t stream) {
    KA_CHECK(m >= 0 && dim > 0, "ka_scatter_rows: bad sizes m=%d dim=%d", m, dim);
    if (m == 0) return 0;
    dim3 grid(m), block(256);
    if (src_dtype == KA_F32)
        hipLaunchKernelGGL(scatter_rows_kernel<float>, grid, block, 0, stream, (const float*)src, rows, out, dim);
    else if (src_dtype == KA_BF16)
        hipLaunchKernelGGL(scatter_rows_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)src, rows, out, dim);
    else
        KA_CHECK(false, "ka_scatter_rows: unsupported dtype %d", src_dtype);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// LayerNorm over the last axis, statistics in fp32, two passes (mean, then the
// variance of the centred values). `rows` (optional) selects input rows, which
// fuses the gather of the wanted positions into the final norm.
// ----------------------------------------------------------------------------
constexpr int LN_THREADS = 256;

__device__ __forceinline__ float block_sum_256(float v, float* smem) {
    v = ka_wave_sum(v);
    int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    __syncthreads();
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < LN_THREADS / KA_WAVE; ++w) total += smem[w];
    return total;
}

template <typename TOut>
__global__ void __launch_bounds__(LN_THREADS)
layernorm_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                 const float* __restrict__ gamma, const float* __restrict__ beta, float eps,
                 TOut* __restrict__ out, int dim) {
    __shared__ float smem[LN_THREADS / KA_WAVE];
    int i = blockIdx.x;
    const float* src = x + (size_t)(rows ? rows[i] : i) * dim;
    TOut* dst = out + (size_t)i * dim;
    float s = 0.f;
    for (int d = threadIdx.x; d < dim; d += LN_THREADS) s += src[d];
    float mean = block_sum_256(s, smem) / (float)dim;
    float v = 0.f;
    for (int d = threadIdx.x; d < dim; d += LN_THREADS) {
        float c = src[d] - mean;
        v += c * c;
    }
    float var = block_sum_256(v, smem) / (float)dim;
    float rstd = 1.0f / sqrtf(var + eps);
    for (int d = threadIdx.x; d < dim; d += LN_THREADS) {
        float y = (src[d] - mean) * rstd * gamma[d];
        if (beta) y += beta[d];
        dst[d] = ka_from_float<TOut>(y);
    }
}

// Rows of up to 256 * 4 * ITEMS values: every thread keeps its share of the row in registers, so
// the row is read once.
template <typename TOut, int ITEMS>
__global__ void __launch_bounds__(LN_THREADS)
layernorm_regs_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                      const float* __restrict__ gamma, const float* __restrict__ beta, float eps,
                      TOut* __restrict__ out, int dim) {
    typedef __attribute__((ext_vector_type(4))) float floatx4;
    __shared__ float smem[LN_THREADS / KA_WAVE];
    int i = blockIdx.x;
    const float* src = x + (size_t)(rows ? rows[i] : i) * dim;
    TOut* dst = out + (size_t)i * dim;
    // (every load unconditional, from a place moved inside the row; a load under a branch would
    // make the compiler wait for each before the next is asked for)
    floatx4 v[ITEMS], g[ITEMS], b[ITEMS];
    float s = 0.f;
    const bool beta_vec = beta && (reinterpret_cast<uintptr_t>(beta) % 16 == 0);
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        int d = min((j * LN_THREADS + (int)threadIdx.x) * 4, dim - 4);
        v[j] = *reinterpret_cast<const floatx4*>(src + d);
        g[j] = *reinterpret_cast<const floatx4*>(gamma + d);
        b[j] = beta_vec ? *reinterpret_cast<const floatx4*>(beta + d) : floatx4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        int d = (j * LN_THREADS + threadIdx.x) * 4;
        if (d >= dim) v[j] = floatx4{0.f, 0.f, 0.f, 0.f};
        if (beta && !beta_vec && d < dim) b[j] = floatx4{beta[d], beta[d + 1], beta[d + 2], beta[d + 3]};
        s += (v[j][0] + v[j][1]) + (v[j][2] + v[j][3]);
    }
    float mean = block_sum_256(s, smem) / (float)dim;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        int d = (j * LN_THREADS + threadIdx.x) * 4;
        if (d < dim) {
#pragma unroll
            for (int e = 0; e < 4; ++e) q += (v[j][e] - mean) * (v[j][e] - mean);
        }
    }
    float rstd = 1.0f / sqrtf(block_sum_256(q, smem) / (float)dim + eps);
    const bool out_vec = reinterpret_cast<uintptr_t>(dst) % (4 * sizeof(TOut)) == 0;      // (dim is a multiple of 4)
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        int d = (j * LN_THREADS + threadIdx.x) * 4;
        if (d < dim) {
            TOut y[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = ka_from_float<TOut>((v[j][e] - mean) * rstd * g[j][e] + b[j][e]);
            if (out_vec) {
                typedef TOut __attribute__((ext_vector_type(4))) out4;
                *reinterpret_cast<out4*>(dst + d) = out4{y[0], y[1], y[2], y[3]};
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) dst[d + e] = y[e];
            }
        }
    }
}

KA_API int ka_layernorm(const float* x, const int* rows, const float* gamma, const float* beta,
                        float eps, void* out, int out_dtype, int n, int dim, hipStream_t stream) {
    KA_CHECK(n >= 0 && dim > 0, "ka_layernorm: bad sizes n=%d dim=%d", n, dim);
    KA_CHECK(eps >= 0.f, "ka_layernorm: negative eps");
    if (n == 0) return 0;
    dim3 grid(n), block(LN_THREADS);
    KA_CHECK(out_dtype == KA_F32 || out_dtype == KA_BF16, "ka_layernorm: unsupported out dtype %d", out_dtype);
    const bool aligned = dim % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)gamma % 16 == 0;
    if (aligned && dim <= LN_THREADS * 4 * 4) {
        // (as many loads per thread as the row needs: 1, 2 or 4 of 16 bytes)
#define KA_LN_REGS(ITEMS)                                                                                                     \
    if (out_dtype == KA_F32)                                                                                                  \
        hipLaunchKernelGGL((layernorm_regs_kernel<float, ITEMS>), grid, block, 0, stream, x, rows, gamma, beta, eps, (float*)out, dim); \
    else                                                                                                                      \
        hipLaunchKernelGGL((layernorm_regs_kernel<bf16_t, ITEMS>), grid, block, 0, stream, x, rows, gamma, beta, eps, (bf16_t*)out, dim)
        if (dim <= LN_THREADS * 4) { KA_LN_REGS(1); }
        else if (dim <= LN_THREADS * 4 * 2) { KA_LN_REGS(2); }
        else { KA_LN_REGS(4); }
#undef KA_LN_REGS
    } else if (out_dtype == KA_F32) {
        hipLaunchKernelGGL(layernorm_kernel<float>, grid, block, 0, stream, x, rows, gamma, beta, eps, (float*)out, dim);
    } else {
        hipLaunchKernelGGL(layernorm_kernel<bf16_t>, grid, block, 0, stream, x, rows, gamma, beta, eps, (bf16_t*)out, dim);
    }
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// Rotary position encoding of the first `rot` channels of each head, applied in place to
// the q heads of a fused qkv row, and to the k heads on their way into the paged cache
// together with v. The table row of position p is [cos(p f_0..f_{rot/2-1}), sin(...)] in
// fp32; the rotation is computed in fp32. `interleaved` says which channels form the pair
// that angle i turns: 0 = channel i with channel i + rot/2 (halves), 1 = channel 2i with
// channel 2i + 1.
//
// qkv row: [H*hd q | Hkv*hd k | Hkv*hd v]. Key cache: [pages, Hkv, page_size, hd]; value cache:
// [pages, Hkv, hd, page_size] (transposed inside the page, so that the MFMA attention kernels
// read eight consecutive keys of one channel with a single 16-byte load).
// slots[t] = page * page_size + offset, or < 0 for "do not write" (a layer that
// reads another layer's cache).
// ----------------------------------------------------------------------------
template <typename T>
__global__ void rope_cache_kernel(T* __restrict__ qkv, long row_stride,
                                  const int* __restrict__ positions, const int* __restrict__ slots,
                                  const float* __restrict__ table, T* __restrict__ k_cache,
                                  T* __restrict__ v_cache, int H, int Hkv, int hd, int rot,
                                  int page_size, int rotate, int interleaved) {
    int t = blockIdx.x;
    T* row = qkv + (size_t)t * row_stride;
    int pos = positions[t];
    const float* cs = table + (size_t)pos * rot;
    int half = rot / 2;
    // q heads: rotate in place. One thread per (head, pair).
    if (rotate) {
        for (int idx = threadIdx.x; idx < H * half; idx += blockDim.x) {
            int h = idx / half, i = idx % half;
            T* p = row + h * hd;
            const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
            float a = ka_to_float(p[ia]), b = ka_to_float(p[ib]);
            float c = cs[i], s = cs[half + i];
            p[ia] = ka_from_float<T>(a * c - b * s);
            p[ib] = ka_from_float<T>(b * c + a * s);
        }
    }
    long slot = slots ? slots[t] : -1;
    if (slot < 0) return;
    long page = slot / page_size, off = slot % page_size;
    const T* krow = row + (size_t)H * hd;
    const T* vrow = krow + (size_t)Hkv * hd;
    for (int idx = threadIdx.x; idx < Hkv * hd; idx += blockDim.x) {
        int h = idx / hd, d = idx % hd;
        size_t dst = (((size_t)page * Hkv + h) * page_size + off) * hd + d;
        float kv = ka_to_float(krow[idx]);
        if (rotate && d < rot) {
            const int i = interleaved ? d / 2 : (d < half ? d : d - half);
            const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
            float a = ka_to_float(krow[h * hd + ia]), b = ka_to_float(krow[h * hd + ib]);
            float c = cs[i], s = cs[half + i];
            kv = d == ia ? a * c - b * s : b * c + a * s;
        }
        k_cache[dst] = ka_from_float<T>(kv);
        size_t vdst = (((size_t)page * Hkv + h) * hd + d) * page_size + off;
        v_cache[vdst] = vrow[idx];
    }
}

KA_API int ka_rope_cache(void* qkv, int dtype, long row_stride, const int* positions,
                         const int* slots, const float* table, int table_rows, void* k_cache,
                         void* v_cache, int n, int H, int Hkv, int hd, int rot, int page_size,
                         int interleaved, hipStream_t stream) {
    KA_CHECK(n >= 0 && H > 0 && Hkv > 0 && hd > 0, "ka_rope_cache: bad sizes");
    KA_CHECK(interleaved == 0 || interleaved == 1, "ka_rope_cache: pairing must be 0 (halves) or 1 (interleaved)");
    KA_CHECK(rot >= 0 && rot <= hd && rot % 2 == 0, "ka_rope_cache: rotary dim %d must be even and <= head dim %d", rot, hd);
    KA_CHECK(row_stride >= (long)(H + 2 * Hkv) * hd, "ka_rope_cache: row stride %ld too small", row_stride);
    KA_CHECK(page_size > 0, "ka_rope_cache: page size %d", page_size);
    KA_CHECK(rot == 0 || (table != nullptr && table_rows > 0), "ka_rope_cache: rotary table missing");
    if (n == 0) return 0;
    dim3 grid(n), block(256);
    int rotate = rot > 0;
    if (dtype == KA_F32)
        hipLaunchKernelGGL(rope_cache_kernel<float>, grid, block, 0, stream, (float*)qkv, row_stride, positions, slots,
                           table, (float*)k_cache, (float*)v_cache, H, Hkv, hd, rot, page_size, rotate, interleaved);
    else if (dtype == KA_BF16)
        hipLaunchKernelGGL(rope_cache_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)qkv, row_stride, positions, slots,
                           table, (bf16_t*)k_cache, (bf16_t*)v_cache, H, Hkv, hd, rot, page_size, rotate, interleaved);
    else
        KA_CHECK(false, "ka_rope_cache: unsupported dtype %d", dtype);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// Learned position vectors: x[t, :] += table[places[t], :] in fp32 (a place outside the table
// adds nothing).
// ----------------------------------------------------------------------------
template <typename T>
__global__ void add_table_rows_kernel(const T* __restrict__ table, int table_rows, const int* __restrict__ places,
                                      float* __restrict__ x, int dim) {
    const int t = blockIdx.x;
    const int p = places[t];
    if ((unsigned)p >= (unsigned)table_rows) return;
    const T* src = table + (size_t)p * dim;
    float* dst = x + (size_t)t * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) dst[d] += ka_to_float(src[d]);
}

KA_API int ka_add_table_rows(const void* table, int table_dtype, int table_rows, const int* places, float* x, int n,
                             int dim, hipStream_t stream) {
    KA_CHECK(n >= 0 && dim > 0 && table_rows > 0, "ka_add_table_rows: bad sizes n=%d dim=%d rows=%d", n, dim, table_rows);
    if (n == 0) return 0;
    dim3 grid(n), block(256);
    if (table_dtype == KA_F32)
        hipLaunchKernelGGL(add_table_rows_kernel<float>, grid, block, 0, stream, (const float*)table, table_rows, places, x, dim);
    else if (table_dtype == KA_BF16)
        hipLaunchKernelGGL(add_table_rows_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)table, table_rows, places, x, dim);
    else
        KA_CHECK(false, "ka_add_table_rows: unsupported table dtype %d", table_dtype);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// fp32 rows into a range of columns of wider rows of the activation type: dst[t, :dim] = src[t, :]
// with dst rows `dst_stride` apart (the caller points dst at the first column of the range).
// Two such calls lay two streams side by side as the input of one linear.
// ----------------------------------------------------------------------------
template <typename T>
__global__ void cast_columns_kernel(const float* __restrict__ src, T* __restrict__ dst, long dst_stride, int dim) {
    const int t = blockIdx.x;
    const float* s = src + (size_t)t * dim;
    T* d = dst + (size_t)t * dst_stride;
    for (int c = threadIdx.x; c < dim; c += blockDim.x) d[c] = ka_from_float<T>(s[c]);
}

KA_API int ka_cast_columns(const float* src, void* dst, int dst_dtype, long dst_stride, int n, int dim, hipStream_t stream) {
    KA_CHECK(n >= 0 && dim > 0 && dst_stride >= dim, "ka_cast_columns: bad sizes n=%d dim=%d stride=%ld", n, dim, dst_stride);
    if (n == 0) return 0;
    dim3 grid(n), block(256);
    if (dst_dtype == KA_F32)
        hipLaunchKernelGGL(cast_columns_kernel<float>, grid, block, 0, stream, src, (float*)dst, dst_stride, dim);
    else if (dst_dtype == KA_BF16)
        hipLaunchKernelGGL(cast_columns_kernel<bf16_t>, grid, block, 0, stream, src, (bf16_t*)dst, dst_stride, dim);
    else
        KA_CHECK(false, "ka_cast_columns: unsupported dtype %d", dst_dtype);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// x += scale * delta over fp32 buffers of one length (a block's branch outputs, summed in delta,
// enter the residual stream with a weight).
// ----------------------------------------------------------------------------
__global__ void add_scaled_kernel(float* __restrict__ x, const float* __restrict__ delta, float scale, long count) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) x[i] = fmaf(scale, delta[i], x[i]);
}

KA_API int ka_add_scaled(float* x, const float* delta, float scale, long count, hipStream_t stream) {
    KA_CHECK(count >= 0 && (count + 255) / 256 < (1L << 31), "ka_add_scaled: bad count %ld", count);
    if (count == 0) return 0;
    hipLaunchKernelGGL(add_scaled_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, x, delta, scale, count);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// Two LayerNorms of the same fp32 rows with gains and shifts of their own (a block whose two
// branches each normalise the block's input), the row read once for both: the mean and variance
// are the same, only gain and shift differ. Optionally, before that, x += scale * delta, the sum of the
// branch outputs of the block before, and, whether added or not, delta is cleared for the branches of
// this block to add into. Without gains (gamma1 null) only that first part runs.
// ----------------------------------------------------------------------------
template <typename TOut>
__global__ void __launch_bounds__(LN_THREADS)
layernorm_pair_kernel(float* __restrict__ x, float* __restrict__ delta, float scale, int apply, int clear,
                      const float* __restrict__ gamma1, const float* __restrict__ beta1,
                      const float* __restrict__ gamma2, const float* __restrict__ beta2, float eps,
                      TOut* __restrict__ out1, TOut* __restrict__ out2, int dim) {
    __shared__ float smem[LN_THREADS / KA_WAVE];
    const int i = blockIdx.x;
    float* row = x + (size_t)i * dim;
    float* drow = delta ? delta + (size_t)i * dim : nullptr;
    float s = 0.f;
    for (int d = threadIdx.x; d < dim; d += LN_THREADS) {
        float v = row[d];
        if (drow) {
            if (apply) {
                v = fmaf(scale, drow[d], v);
                row[d] = v;
            }
            if (clear) drow[d] = 0.f;
        }
        s += v;
    }
    if (!gamma1) return;
    // (every thread reads back only what it has written itself)
    const float mean = block_sum_256(s, smem) / (float)dim;
    float q = 0.f;
    for (int d = threadIdx.x; d < dim; d += LN_THREADS) {
        const float c = row[d] - mean;
        q += c * c;
    }
    const float rstd = 1.0f / sqrtf(block_sum_256(q, smem) / (float)dim + eps);
    TOut* dst1 = out1 + (size_t)i * dim;
    TOut* dst2 = out2 ? out2 + (size_t)i * dim : nullptr;
    for (int d = threadIdx.x; d < dim; d += LN_THREADS) {
        const float c = (row[d] - mean) * rstd;
        float y = c * gamma1[d];
        if (beta1) y += beta1[d];
        dst1[d] = ka_from_float<TOut>(y);
        if (dst2) {
            float z = c * gamma2[d];
            if (beta2) z += beta2[d];
            dst2[d] = ka_from_float<TOut>(z);
        }
    }
}

// The same for rows of up to 256 * 4 * ITEMS values that are 16-byte aligned: every thread keeps its share of the
// row in registers, so the row (and what is added to it) is read once.
template <typename TOut, int ITEMS>
__global__ void __launch_bounds__(LN_THREADS)
layernorm_pair_regs_kernel(float* __restrict__ x, float* __restrict__ delta, float scale, int apply, int clear,
                           const float* __restrict__ gamma1, const float* __restrict__ beta1,
                           const float* __restrict__ gamma2, const float* __restrict__ beta2, float eps,
                           TOut* __restrict__ out1, TOut* __restrict__ out2, int dim) {
    typedef __attribute__((ext_vector_type(4))) float floatx4;
    typedef TOut __attribute__((ext_vector_type(4))) out4;
    __shared__ float smem[LN_THREADS / KA_WAVE];
    const int i = blockIdx.x;
    float* row = x + (size_t)i * dim;
    float* drow = delta ? delta + (size_t)i * dim : nullptr;
    floatx4 v[ITEMS];
    float s = 0.f;
    // (loads first, all of them in flight together; then the arithmetic and the stores)
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const int d = min((j * LN_THREADS + (int)threadIdx.x) * 4, dim - 4);
        v[j] = *reinterpret_cast<const floatx4*>(row + d);
    }
    if (drow && apply) {
        floatx4 a[ITEMS];
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            const int d = min((j * LN_THREADS + (int)threadIdx.x) * 4, dim - 4);
            a[j] = *reinterpret_cast<const floatx4*>(drow + d);
        }
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            const int d = (j * LN_THREADS + threadIdx.x) * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[j][e] = fmaf(scale, a[j][e], v[j][e]);
            if (d < dim) *reinterpret_cast<floatx4*>(row + d) = v[j];
        }
    }
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const int d = (j * LN_THREADS + threadIdx.x) * 4;
        if (d >= dim) v[j] = floatx4{0.f, 0.f, 0.f, 0.f};
        else if (drow && clear) *reinterpret_cast<floatx4*>(drow + d) = floatx4{0.f, 0.f, 0.f, 0.f};
        s += (v[j][0] + v[j][1]) + (v[j][2] + v[j][3]);
    }
    if (!gamma1) return;
    const float mean = block_sum_256(s, smem) / (float)dim;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const int d = (j * LN_THREADS + threadIdx.x) * 4;
        if (d < dim) {
#pragma unroll
            for (int e = 0; e < 4; ++e) q += (v[j][e] - mean) * (v[j][e] - mean);
        }
    }
    const float rstd = 1.0f / sqrtf(block_sum_256(q, smem) / (float)dim + eps);
    TOut* dst1 = out1 + (size_t)i * dim;
    TOut* dst2 = out2 ? out2 + (size_t)i * dim : nullptr;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const int d = (j * LN_THREADS + threadIdx.x) * 4;
        if (d < dim) {
            const floatx4 g1 = *reinterpret_cast<const floatx4*>(gamma1 + d);
            const floatx4 b1 = beta1 ? *reinterpret_cast<const floatx4*>(beta1 + d) : floatx4{0.f, 0.f, 0.f, 0.f};
            out4 y;
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = ka_from_float<TOut>((v[j][e] - mean) * rstd * g1[e] + b1[e]);
            *reinterpret_cast<out4*>(dst1 + d) = y;
            if (dst2) {
                const floatx4 g2 = *reinterpret_cast<const floatx4*>(gamma2 + d);
                const floatx4 b2 = beta2 ? *reinterpret_cast<const floatx4*>(beta2 + d) : floatx4{0.f, 0.f, 0.f, 0.f};
                out4 z;
#pragma unroll
                for (int e = 0; e < 4; ++e) z[e] = ka_from_float<TOut>((v[j][e] - mean) * rstd * g2[e] + b2[e]);
                *reinterpret_cast<out4*>(dst2 + d) = z;
            }
        }
    }
}

// clear: delta is zeroed (after it was added, if apply), for branches that add into it.
KA_API int ka_layernorm_pair(float* x, float* delta, float scale, int apply, int clear, const float* gamma1,
                             const float* beta1, const float* gamma2, const float* beta2, float eps, void* out1, void* out2,
                             int out_dtype, int n, int dim, hipStream_t stream) {
    KA_CHECK(n >= 0 && dim > 0 && eps >= 0.f, "ka_layernorm_pair: bad sizes n=%d dim=%d", n, dim);
    KA_CHECK((!apply && !clear) || delta, "ka_layernorm_pair: nothing to add or clear");
    KA_CHECK(gamma1 || (delta && (apply || clear)), "ka_layernorm_pair: nothing to do");
    KA_CHECK(!gamma1 || out1, "ka_layernorm_pair: the first norm has no output");
    KA_CHECK((out2 != nullptr) == (gamma2 != nullptr), "ka_layernorm_pair: the second norm needs gains and an output");
    KA_CHECK(out_dtype == KA_F32 || out_dtype == KA_BF16, "ka_layernorm_pair: unsupported out dtype %d", out_dtype);
    if (n == 0) return 0;
    dim3 grid(n), block(LN_THREADS);
    auto aligned = [](const void* p) { return p == nullptr || (uintptr_t)p % 16 == 0; };
    const bool regs = dim % 4 == 0 && dim <= LN_THREADS * 4 * 4 && aligned(x) && aligned(delta) && aligned(gamma1) && aligned(beta1) &&
                      aligned(gamma2) && aligned(beta2) && aligned(out1) && aligned(out2);
#define KA_LNP(KERNEL, TOUT)                                                                                              \
    hipLaunchKernelGGL((KERNEL), grid, block, 0, stream, x, delta, scale, apply, clear, gamma1, beta1, gamma2, beta2, eps, \
                       (TOUT*)out1, (TOUT*)out2, dim)
#define KA_LNP_REGS(ITEMS)                                                        \
    if (out_dtype == KA_F32) { KA_LNP((layernorm_pair_regs_kernel<float, ITEMS>), float); } \
    else { KA_LNP((layernorm_pair_regs_kernel<bf16_t, ITEMS>), bf16_t); }
    if (regs && dim <= LN_THREADS * 4) { KA_LNP_REGS(1) }
    else if (regs && dim <= LN_THREADS * 4 * 2) { KA_LNP_REGS(2) }
    else if (regs) { KA_LNP_REGS(4) }
    else if (out_dtype == KA_F32) { KA_LNP(layernorm_pair_kernel<float>, float); }
    else { KA_LNP(layernorm_pair_kernel<bf16_t>, bf16_t); }
#undef KA_LNP_REGS
#undef KA_LNP
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// Unit-norm queries and keys + paged cache write, for attention without a rotation whose queries and
// keys are divided, head by head, by their root mean square (x / sqrt(mean(x^2) + eps), no gain;
// arithmetic in fp32), and whose values may have another size than its keys.
//
// qkv row: [H*hd q | Hkv*hd k | Hkv*hdv v]. q and k are normalised in place (normalise != 0); k and v
// then go into the cache: keys [pages, Hkv, page_size, hd], values [pages, Hkv, hdv, page_size].
// slots as for ka_rope_cache. A wave per head of a token, four heads a workgroup.
// ----------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
unit_norm_cache_kernel(T* __restrict__ qkv, long row_stride, const int* __restrict__ slots, T* __restrict__ k_cache,
                       T* __restrict__ v_cache, int H, int Hkv, int hd, int hdv, int page_size, float eps, int normalise,
                       int with_values) {
    // a wave per head of a token: the query heads, then the key heads, then (with_values) the value heads
    const int t = blockIdx.x;
    const int lane = threadIdx.x % KA_WAVE;
    const int h = blockIdx.y * (blockDim.x / KA_WAVE) + threadIdx.x / KA_WAVE;
    if (h >= H + (with_values ? 2 : 1) * Hkv) return;
    T* row = qkv + (size_t)t * row_stride;
    const long slot = slots ? slots[t] : -1;
    const long page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
    if (h >= H + Hkv) {
        if (slot < 0) return;
        const int g = h - H - Hkv;
        const T* vrow = row + (size_t)(H + Hkv) * hd + (size_t)g * hdv;
        T* dst = v_cache + (((size_t)page * Hkv + g) * hdv) * page_size + off;
        for (int d = lane; d < hdv; d += KA_WAVE) dst[(size_t)d * page_size] = vrow[d];
        return;
    }
    T* p = row + (size_t)h * hd;
    const bool key = h >= H;
    if (!normalise && !(key && slot >= 0)) return;
    T* kdst = key && slot >= 0 ? k_cache + (((size_t)page * Hkv + (h - H)) * page_size + off) * hd : nullptr;
    if (hd <= KA_WAVE) {
        // the whole head in one load a lane
        const float v = lane < hd ? ka_to_float(p[lane]) : 0.f;
        const float rinv = normalise ? 1.0f / sqrtf(ka_wave_sum(v * v) / (float)hd + eps) : 1.f;
        if (lane < hd) {
            const T y = ka_from_float<T>(v * rinv);
            if (normalise) p[lane] = y;
            if (kdst) kdst[lane] = y;
        }
        return;
    }
    float rinv = 1.f;
    if (normalise) {
        float ss = 0.f;
        for (int d = lane; d < hd; d += KA_WAVE) {
            const float v = ka_to_float(p[d]);
            ss = fmaf(v, v, ss);
        }
        rinv = 1.0f / sqrtf(ka_wave_sum(ss) / (float)hd + eps);
    }
    for (int d = lane; d < hd; d += KA_WAVE) {
        const T y = ka_from_float<T>(ka_to_float(p[d]) * rinv);
        if (normalise) p[d] = y;
        if (kdst) kdst[d] = y;
    }
}

// The same for bf16 heads of a multiple of 8 channels on 16-byte aligned rows: a lane holds a 16-byte chunk of a head,
// LPH lanes (the next power of two of hd / 8) a head, 64 / LPH heads a wave; the sum of squares meets inside those lanes.
// Query and key heads only (the values go run by run, or through the kernel above).
template <int LPH>
__global__ void __launch_bounds__(256)
unit_norm_cache_chunks_kernel(bf16_t* __restrict__ qkv, long row_stride, const int* __restrict__ slots,
                              bf16_t* __restrict__ k_cache, int H, int Hkv, int hd, int page_size, float eps, int normalise) {
    typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
    const int t = blockIdx.x;
    const int lane = threadIdx.x % KA_WAVE;
    const int h = (blockIdx.y * (blockDim.x / KA_WAVE) + threadIdx.x / KA_WAVE) * (KA_WAVE / LPH) + lane / LPH;
    const int c = (lane % LPH) * 8;
    const bool live = h < H + Hkv && c < hd;
    bf16_t* p = qkv + (size_t)t * row_stride + (size_t)(live ? h : 0) * hd + (live ? c : 0);
    bf16x8 v = *reinterpret_cast<const bf16x8*>(p);
    float f[8], ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        f[e] = live ? (float)v[e] : 0.f;
        ss = fmaf(f[e], f[e], ss);
    }
    ss = ka_lanes_reduce<1, LPH>(ss, KaSum{});
    if (!live) return;
    const float rinv = normalise ? 1.0f / sqrtf(ss / (float)hd + eps) : 1.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (bf16_t)(f[e] * rinv);
    if (normalise) *reinterpret_cast<bf16x8*>(p) = v;
    const long slot = slots ? slots[t] : -1;
    if (h >= H && slot >= 0)
        *reinterpret_cast<bf16x8*>(k_cache + (((size_t)(slot / page_size) * Hkv + (h - H)) * page_size + slot % page_size) * hd + c) = v;
}

// The values of runs of tokens into the cache. A run is `count` neighbouring tokens of the packed batch (at most a
// page's worth); one that fills a page of its row in order (count == page_size, the first at a page's start, the
// slots consecutive) is turned through LDS and leaves as the page's contiguous [hdv][page_size] block; any other
// run goes token by token. One workgroup per (run, kv head).
constexpr int UN_MAX_TILE = 16 * 520;            // page 16, value heads of up to 512 channels (+ padding)

template <typename T>
__global__ void __launch_bounds__(256)
value_cache_runs_kernel(const T* __restrict__ qkv, long row_stride, long v_offset, const int* __restrict__ slots,
                        const int* __restrict__ run_first, const int* __restrict__ run_count, T* __restrict__ v_cache,
                        int Hkv, int hdv, int page_size) {
    __shared__ T tile[UN_MAX_TILE];
    const int count = run_count[blockIdx.x];
    if (count <= 0) return;
    const int first = run_first[blockIdx.x], g = blockIdx.y;
    const int s0 = slots[first];
    const int pitch = hdv + 2;
    const bool whole = count == page_size && page_size == 16 && s0 >= 0 && s0 % page_size == 0 &&
                       slots[first + count - 1] == s0 + count - 1 && page_size * pitch <= UN_MAX_TILE;
    if (whole) {
        for (int idx = threadIdx.x; idx < page_size * hdv; idx += blockDim.x) {
            const int i = idx / hdv, d = idx % hdv;
            tile[i * pitch + d] = qkv[(size_t)(first + i) * row_stride + v_offset + (size_t)g * hdv + d];
        }
        __syncthreads();
        T* dst = v_cache + (((size_t)(s0 / page_size) * Hkv + g) * hdv) * page_size;
        for (int idx = threadIdx.x; idx < page_size * hdv; idx += blockDim.x) {
            const int d = idx / page_size, i = idx % page_size;
            dst[idx] = tile[i * pitch + d];
        }
        return;
    }
    for (int idx = threadIdx.x; idx < count * hdv; idx += blockDim.x) {
        const int i = idx / hdv, d = idx % hdv;
        const long slot = slots[first + i];
        if (slot < 0) continue;
        v_cache[(((size_t)(slot / page_size) * Hkv + g) * hdv + d) * page_size + slot % page_size] =
            qkv[(size_t)(first + i) * row_stride + v_offset + (size_t)g * hdv + d];
    }
}

// run_first / run_count (optional, n_runs of them): the tokens cut into runs, every token in exactly one and none
// longer than a page; the values then go into the cache run by run (whole pages as contiguous blocks).
KA_API int ka_unit_norm_cache(void* qkv, int dtype, long row_stride, const int* slots, void* k_cache, void* v_cache,
                              int n, int H, int Hkv, int hd, int hdv, int page_size, float eps, int normalise,
                              const int* run_first, const int* run_count, int n_runs, hipStream_t stream) {
    KA_CHECK(n >= 0 && H > 0 && Hkv > 0 && hd > 0 && hdv > 0, "ka_unit_norm_cache: bad sizes");
    KA_CHECK(row_stride >= (long)(H + Hkv) * hd + (long)Hkv * hdv, "ka_unit_norm_cache: row stride %ld too small", row_stride);
    KA_CHECK(page_size > 0 && eps >= 0.f, "ka_unit_norm_cache: page size %d, eps %g", page_size, eps);
    KA_CHECK(slots == nullptr || (k_cache && v_cache), "ka_unit_norm_cache: cache tensors missing");
    if (n == 0) return 0;
    KA_CHECK((H + 2 * Hkv + 3) / 4 <= 65535, "ka_unit_norm_cache: too many heads");
    const bool by_runs = slots && run_first && run_count && n_runs > 0 && Hkv <= 65535;
    // (with the values written run by run, the first launch ends with the key heads: the kernel passes over heads
    // behind H + 2 Hkv, so it is told of no value heads at all by way of its grid)
    dim3 grid(n, ((by_runs ? H + Hkv : H + 2 * Hkv) + 3) / 4), block(256);
    if (by_runs) {
        dim3 rgrid(n_runs, Hkv);
        const long v_offset = (long)(H + Hkv) * hd;
        if (dtype == KA_F32)
            hipLaunchKernelGGL(value_cache_runs_kernel<float>, rgrid, block, 0, stream, (const float*)qkv, row_stride, v_offset,
                               slots, run_first, run_count, (float*)v_cache, Hkv, hdv, page_size);
        else if (dtype == KA_BF16)
            hipLaunchKernelGGL(value_cache_runs_kernel<bf16_t>, rgrid, block, 0, stream, (const bf16_t*)qkv, row_stride, v_offset,
                               slots, run_first, run_count, (bf16_t*)v_cache, Hkv, hdv, page_size);
    }
    // bf16 heads in 16-byte chunks where rows and heads are aligned for it (the values then go run by run, or, without
    // runs, through a launch of the plain kernel that starts behind the key heads: here the plain kernel does it all)
    const int chunks = hd / 8;
    if (dtype == KA_BF16 && by_runs && hd % 8 == 0 && chunks <= 64 && row_stride % 8 == 0 && (uintptr_t)qkv % 16 == 0 &&
        (uintptr_t)k_cache % 16 == 0) {
        int lph = 1;
        while (lph < chunks) lph *= 2;
        const int heads_per_block = 4 * (KA_WAVE / lph);
        dim3 cgrid(n, (H + Hkv + heads_per_block - 1) / heads_per_block);
#define KA_UN_CHUNKS(LPH)                                                                                                  \
    if (lph == LPH)                                                                                                        \
        hipLaunchKernelGGL(unit_norm_cache_chunks_kernel<LPH>, cgrid, block, 0, stream, (bf16_t*)qkv, row_stride, slots,   \
                           (bf16_t*)k_cache, H, Hkv, hd, page_size, eps, normalise)
        KA_UN_CHUNKS(1); KA_UN_CHUNKS(2); KA_UN_CHUNKS(4); KA_UN_CHUNKS(8); KA_UN_CHUNKS(16); KA_UN_CHUNKS(32); KA_UN_CHUNKS(64);
#undef KA_UN_CHUNKS
        KA_LAUNCH_CHECK();
        return 0;
    }
    if (dtype == KA_F32)
        hipLaunchKernelGGL(unit_norm_cache_kernel<float>, grid, block, 0, stream, (float*)qkv, row_stride, slots,
                           (float*)k_cache, (float*)v_cache, H, Hkv, hd, hdv, page_size, eps, normalise, by_runs ? 0 : 1);
    else if (dtype == KA_BF16)
        hipLaunchKernelGGL(unit_norm_cache_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)qkv, row_stride, slots,
                           (bf16_t*)k_cache, (bf16_t*)v_cache, H, Hkv, hd, hdv, page_size, eps, normalise, by_runs ? 0 : 1);
    else
        KA_CHECK(false, "ka_unit_norm_cache: unsupported dtype %d", dtype);
    KA_LAUNCH_CHECK();
    return 0;
}
