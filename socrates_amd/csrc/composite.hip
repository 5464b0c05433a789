// Kernels of layers that norm their results and average over depth, of window attention with biases,
// whole-projection norms, rotations over interleaved pairs, turned values and pooled blocks, of linear
// attention with a decay per head or per key channel and token, and of the gelu-gated feed-forward.
//
// Statistics, angles, decays and their logarithms, the recurrence and its state, the residual sum and
// the weighted sum over depth are float32 whatever the compute dtype; a value is rounded once, where it
// is stored in the compute dtype.
#include "common.h"
#include "recurrent.h"

__device__ __forceinline__ float cmp_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float cmp_silu(float x) { return x * cmp_sigmoid(x); }

// ---- residual += norm(y) * gain, and the sum in the compute dtype ---------------------------------------
// One workgroup per row. y: the compute dtype or float32. With kept ([total, n] float32, n = rows * d): the sum is the
// layer's result, filed as kept[count], and what goes on (into residual and out) is sum over j <= count of w[j] kept[j],
// in that order (the weighted sum over depth, below, in the same kernel).
template <typename T, typename Y>
__global__ void __launch_bounds__(256)
norm_add_cast_kernel(float* __restrict__ residual, const Y* __restrict__ y, const float* __restrict__ gain, float eps,
                     T* __restrict__ out, int d, float* __restrict__ kept, int count, const float* __restrict__ w, size_t n) {
    __shared__ float scratch[16];
    const size_t row = (size_t)blockIdx.x * d;
    float ss = 0.f;
    for (int c = threadIdx.x; c < d; c += 256) { const float v = to_float(y[row + c]); ss = fmaf(v, v, ss); }
    ss = block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)d + eps);
    for (int c = threadIdx.x; c < d; c += 256) {
        float r = residual[row + c] + to_float(y[row + c]) * inv * gain[c];
        if (kept) {                                        // the layer's result is filed, the weighted sum over depth goes on
            kept[(size_t)count * n + row + c] = r;
            float acc = 0.f;
            for (int j = 0; j < count; ++j) acc = fmaf(w[j], kept[(size_t)j * n + row + c], acc);
            r = fmaf(w[count], r, acc);
        }
        residual[row + c] = r;
        if (out) out[row + c] = from_float<T>(r);
    }
}

// The same for rows of up to 256 * 8 * C elements, a multiple of 8: a thread keeps its C runs of 8 in registers
// between the sum of squares and the sum into the stream.
template <typename T, typename Y, int C>
__global__ void __launch_bounds__(256)
norm_add_cast_vec8_kernel(float* __restrict__ residual, const Y* __restrict__ y, const float* __restrict__ gain, float eps,
                          T* __restrict__ out, int d, float* __restrict__ kept, int count, const float* __restrict__ w, size_t n) {
    __shared__ float scratch[16];
    const size_t row = (size_t)blockIdx.x * d;
    float v[C][8];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int at = (threadIdx.x + c * 256) * 8;
        if (at < d) {
            VecLoad<Y, 8>::load(y + row + at, v[c]);
#pragma unroll
            for (int e = 0; e < 8; ++e) ss = fmaf(v[c][e], v[c][e], ss);
        }
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)d + eps);
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int at = (threadIdx.x + c * 256) * 8;
        if (at < d) {
            float r[8], g[8];
            VecLoad<float, 8>::load(residual + row + at, r);
            VecLoad<float, 8>::load(gain + at, g);
#pragma unroll
            for (int e = 0; e < 8; ++e) r[e] += v[c][e] * inv * g[e];
            if (kept) {
                float* own = kept + (size_t)count * n + row + at;
                *reinterpret_cast<float4*>(own) = make_float4(r[0], r[1], r[2], r[3]);
                *reinterpret_cast<float4*>(own + 4) = make_float4(r[4], r[5], r[6], r[7]);
                float acc[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] = 0.f;
                for (int j = 0; j < count; ++j) {
                    float t[8];
                    VecLoad<float, 8>::load(kept + (size_t)j * n + row + at, t);
                    const float wj = w[j];
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[e] = fmaf(wj, t[e], acc[e]);
                }
                const float wc = w[count];
#pragma unroll
                for (int e = 0; e < 8; ++e) r[e] = fmaf(wc, r[e], acc[e]);
            }
            *reinterpret_cast<float4*>(residual + row + at) = make_float4(r[0], r[1], r[2], r[3]);
            *reinterpret_cast<float4*>(residual + row + at + 4) = make_float4(r[4], r[5], r[6], r[7]);
            if (out) {
                if constexpr (sizeof(T) == 2) {
                    uint4 pk;
                    pk.x = pack_bf16x2(r[0], r[1]); pk.y = pack_bf16x2(r[2], r[3]);
                    pk.z = pack_bf16x2(r[4], r[5]); pk.w = pack_bf16x2(r[6], r[7]);
                    *reinterpret_cast<uint4*>(out + row + at) = pk;
                } else {
                    float* of = reinterpret_cast<float*>(out + row + at);
                    *reinterpret_cast<float4*>(of) = make_float4(r[0], r[1], r[2], r[3]);
                    *reinterpret_cast<float4*>(of + 4) = make_float4(r[4], r[5], r[6], r[7]);
                }
            }
        }
    }
}

SOC_EXPORT int soc_norm_add_cast(float* residual, const void* y, int y_f32, const float* gain, float eps, void* out, int N,
                                 int d, float* kept, int count, const float* w, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (d < 1 || (kept && (count < 1 || !w))) return (int)hipErrorInvalidValue;
    const size_t n = (size_t)N * d;
#define SOC_NAC(T, Y)                                                                                                                \
    do {                                                                                                                             \
        if (d % 8 == 0 && d <= 2048) hipLaunchKernelGGL((norm_add_cast_vec8_kernel<T, Y, 1>), dim3(N), dim3(256), 0, stream, residual, (const Y*)y, gain, eps, (T*)out, d, kept, count, w, n);      \
        else if (d % 8 == 0 && d <= 4096) hipLaunchKernelGGL((norm_add_cast_vec8_kernel<T, Y, 2>), dim3(N), dim3(256), 0, stream, residual, (const Y*)y, gain, eps, (T*)out, d, kept, count, w, n); \
        else if (d % 8 == 0 && d <= 8192) hipLaunchKernelGGL((norm_add_cast_vec8_kernel<T, Y, 4>), dim3(N), dim3(256), 0, stream, residual, (const Y*)y, gain, eps, (T*)out, d, kept, count, w, n); \
        else hipLaunchKernelGGL((norm_add_cast_kernel<T, Y>), dim3(N), dim3(256), 0, stream, residual, (const Y*)y, gain, eps, (T*)out, d, kept, count, w, n);                                     \
    } while (0)
    if (dtype == 0) SOC_NAC(float, float);
    else if (y_f32) SOC_NAC(bf16, float);
    else SOC_NAC(bf16, bf16);
#undef SOC_NAC
    return soc_last_error();
}

// ---- the first of the results by depth: kept[0] <- residual, and the stream in the compute dtype ----------------
template <typename T>
__global__ void depth_begin_kernel(const float* __restrict__ residual, float* __restrict__ kept, T* __restrict__ out, size_t n) {
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
        const float v = residual[e];
        kept[e] = v;
        if (out) out[e] = from_float<T>(v);
    }
}

SOC_EXPORT int soc_depth_begin(const float* residual, float* kept, void* out, long long n, int dtype, hipStream_t stream) {
    if (n <= 0) return 0;
    const int blocks = (int)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
    if (dtype == 0)
        hipLaunchKernelGGL(depth_begin_kernel<float>, dim3(blocks), dim3(256), 0, stream, residual, kept, (float*)out, (size_t)n);
    else
        hipLaunchKernelGGL(depth_begin_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, residual, kept, (bf16*)out, (size_t)n);
    return soc_last_error();
}

// ---- the weighted sum over depth ----------------------------------------------------------------------------
// kept [total, n] float32: kept[count] <- residual (the layer's own result); residual <- sum over
// j = 0 .. count of w[j] kept[j], in that order; out (if given): the sum in the compute dtype.
template <typename T>
__global__ void depth_average_kernel(float* __restrict__ residual, float* __restrict__ kept, int count, const float* __restrict__ w,
                                     T* __restrict__ out, size_t n) {
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
        const float own = residual[e];
        kept[(size_t)count * n + e] = own;
        float acc = 0.f;
        for (int j = 0; j < count; ++j) acc = fmaf(w[j], kept[(size_t)j * n + e], acc);
        acc = fmaf(w[count], own, acc);
        residual[e] = acc;
        if (out) out[e] = from_float<T>(acc);
    }
}

SOC_EXPORT int soc_depth_average(float* residual, float* kept, int count, const float* w, void* out, long long n, int dtype,
                                 hipStream_t stream) {
    if (n <= 0) return 0;
    if (count < 0) return (int)hipErrorInvalidValue;
    const int blocks = (int)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
    if (dtype == 0)
        hipLaunchKernelGGL(depth_average_kernel<float>, dim3(blocks), dim3(256), 0, stream, residual, kept, count, w, (float*)out, (size_t)n);
    else
        hipLaunchKernelGGL(depth_average_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, residual, kept, count, w, (bf16*)out, (size_t)n);
    return soc_last_error();
}

// ---- biases, norms, rotation over interleaved pairs, turned values, page writes -------------------------------
// x: rows of ld elements that hold, from col_q / col_k / col_v on, Hq heads of D, Hkv heads of D and Hkv heads of
// Dv; bias (or null): float32 [ld], added to those columns. norm 0: none; 1: q and k RMS-normed per head with gains
// [D]; 2: over the whole of q (gain [Hq D]) and the whole of k (gain [Hkv D]); 3: per head behind the rotation, no
// gain. Then elements 2i and 2i + 1 of the
// first 2 * half of every q and k head are turned by position * inv_freq[i] (cosines and sines times magnitude), and (value_freq given) elements 2m and
// 2m + 1 of every v head by position * value_freq[m]. q goes to q_out [N, Hq, P], k and v to the token's place in the
// pools [pages, Hkv, BS, P] (P even), zeros behind D and Dv (Hkv 0: queries only, no pools). grid (tokens, groups of
// per heads); a workgroup's q and k heads pass through LDS (dynamic, per * D floats).
template <typename T>
__global__ void __launch_bounds__(256)
window_prepare_kernel(const T* __restrict__ x, int ld, int col_q, int col_k, int col_v, const float* __restrict__ bias,
                      T* __restrict__ q_out, T* __restrict__ k_pool, T* __restrict__ v_pool, const int* __restrict__ table,
                      int table_width, const int* __restrict__ token_rows, const int* __restrict__ positions,
                      const float* __restrict__ q_gain, const float* __restrict__ k_gain, int norm, float eps,
                      const float* __restrict__ inv_freq, int half, float magnitude, const float* __restrict__ value_freq,
                      int Hq, int Hkv, int D, int Dv, int P, int BS, int per) {
    extern __shared__ float qk[];                          // the workgroup's heads: [per][D]
    __shared__ float scratch[16];
    const int n = blockIdx.x, tid = threadIdx.x;
    const int pos = positions[n];
    const T* row = x + (size_t)n * ld;
    const int nq = Hq * D, nk = Hkv * D;
    // the workgroup's heads among the Hq of q and, behind them, the Hkv of k (a k head brings its v head along)
    const int h_lo = blockIdx.y * per, h_hi = min(Hq + Hkv, h_lo + per);
    if (h_lo >= h_hi) return;
    auto column = [&](int h, int i) { return h < Hq ? col_q + h * D + i : col_k + (h - Hq) * D + i; };
    float iq = 1.f, ik = 1.f;
    if (norm == 2) {
        // the statistics of the whole of q and of k: every workgroup of the token takes them for itself
        float sq = 0.f, sk = 0.f;
        for (int e = tid; e < nq; e += 256) { const float v = to_float(row[col_q + e]) + (bias ? bias[col_q + e] : 0.f); sq = fmaf(v, v, sq); }
        for (int e = tid; e < nk; e += 256) { const float v = to_float(row[col_k + e]) + (bias ? bias[col_k + e] : 0.f); sk = fmaf(v, v, sk); }
        sq = block_sum(sq, scratch);
        sk = block_sum(sk, scratch);
        iq = 1.f / sqrtf(sq / (float)nq + eps);
        ik = 1.f / sqrtf(sk / (float)nk + eps);
    }
    for (int e = tid; e < (h_hi - h_lo) * D; e += 256) {
        const int h = h_lo + e / D, i = e % D;
        const int c = column(h, i);
        float v = to_float(row[c]) + (bias ? bias[c] : 0.f);
        if (norm == 2) v = h < Hq ? v * iq * q_gain[h * D + i] : v * ik * k_gain[(h - Hq) * D + i];
        qk[e] = v;
    }
    __syncthreads();
    if (norm == 1) {
        const int wave = tid / SOC_WAVE, lane = tid % SOC_WAVE;
        for (int h = h_lo + wave; h < h_hi; h += 256 / SOC_WAVE) {
            float* head = qk + (size_t)(h - h_lo) * D;
            const float* gain = h < Hq ? q_gain : k_gain;
            float ss = 0.f;
            for (int i = lane; i < D; i += SOC_WAVE) ss = fmaf(head[i], head[i], ss);
            const float inv = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
            for (int i = lane; i < D; i += SOC_WAVE) head[i] = head[i] * inv * gain[i];
        }
        __syncthreads();
    }
    if (norm == 3) {
        // turned in place, then each head over its root mean square; the writes below then turn nothing
        for (int e = tid; e < (h_hi - h_lo) * half; e += 256) {
            float* head = qk + (size_t)(e / half) * D;
            const int j = e % half;
            float sn, cs;
            sincosf((float)pos * inv_freq[j], &sn, &cs);
            sn *= magnitude; cs *= magnitude;
            const float a = head[2 * j], b = head[2 * j + 1];
            head[2 * j] = a * cs - b * sn;
            head[2 * j + 1] = b * cs + a * sn;
        }
        __syncthreads();
        const int wave = tid / SOC_WAVE, lane = tid % SOC_WAVE;
        for (int h = h_lo + wave; h < h_hi; h += 256 / SOC_WAVE) {
            float* head = qk + (size_t)(h - h_lo) * D;
            float ss = 0.f;
            for (int i = lane; i < D; i += SOC_WAVE) ss = fmaf(head[i], head[i], ss);
            const float inv = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
            for (int i = lane; i < D; i += SOC_WAVE) head[i] = head[i] * inv;
        }
        __syncthreads();
        half = 0;
    }
    const int page = Hkv ? table[(size_t)token_rows[n] * table_width + pos / BS] : 0;
    const size_t place = (size_t)page * Hkv * BS + (size_t)(pos % BS);
    // A thread owns one pair (2j, 2j + 1) of the padded head size and walks heads with it: the pair's angle is taken
    // once (P is even: the pools' head size; 256 / (P / 2) threads share a pair's heads among them).
    const int PP = P / 2, lanes = 256 / PP;                // (P <= 256: at least two threads per pair)
    const int j = tid % PP, g = tid / PP;
    if (g < lanes) {
        float sn = 0.f, cs = 1.f;
        if (j < half) { sincosf((float)pos * inv_freq[j], &sn, &cs); sn *= magnitude; cs *= magnitude; }
        for (int h = h_lo + g; h < h_hi; h += lanes) {
            const float* head = qk + (size_t)(h - h_lo) * D;
            const float a = 2 * j < D ? head[2 * j] : 0.f, b = 2 * j + 1 < D ? head[2 * j + 1] : 0.f;
            const float y0 = j < half ? a * cs - b * sn : a, y1 = j < half ? b * cs + a * sn : b;
            T* dst = h < Hq ? q_out + ((size_t)n * Hq + h) * P : k_pool + (place + (size_t)(h - Hq) * BS) * P;
            dst[2 * j] = from_float<T>(y0);
            dst[2 * j + 1] = from_float<T>(y1);
        }
        // the v heads of the workgroup's k heads
        sn = 0.f; cs = 1.f;
        if (value_freq && 2 * j + 1 < Dv) sincosf((float)pos * value_freq[j], &sn, &cs);
        for (int h = max(h_lo, Hq) - Hq + g; h < h_hi - Hq; h += lanes) {
            const int c = col_v + h * Dv + 2 * j;
            const float a = 2 * j < Dv ? to_float(row[c]) + (bias ? bias[c] : 0.f) : 0.f;
            const float b = 2 * j + 1 < Dv ? to_float(row[c + 1]) + (bias ? bias[c + 1] : 0.f) : 0.f;
            T* dst = v_pool + (place + (size_t)h * BS) * P;
            dst[2 * j] = from_float<T>(a * cs - b * sn);
            dst[2 * j + 1] = from_float<T>(b * cs + a * sn);
        }
    }
}

SOC_EXPORT int soc_window_prepare(const void* x, int ld, int col_q, int col_k, int col_v, const float* bias, void* q_out,
                                  void* k_pool, void* v_pool, const int* table, int table_width, const int* token_rows,
                                  const int* positions, const float* q_gain, const float* k_gain, int norm, float eps,
                                  const float* inv_freq, int half, float magnitude, const float* value_freq, int N, int Hq,
                                  int Hkv, int D, int Dv, int P, int BS, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (D < 1 || Dv < 1 || D > P || Dv > P || P > 256 || P % 2 || 2 * half > D || BS < 1 || norm < 0 || norm > 3 || Hq < 1 || Hkv < 0)
        return (int)hipErrorInvalidValue;
    if (Hkv > 0 && (!k_pool || !v_pool || !table)) return (int)hipErrorInvalidValue;
    if ((norm == 1 || norm == 2) && (!q_gain || !k_gain)) return (int)hipErrorInvalidValue;
    if (half && !inv_freq) return (int)hipErrorInvalidValue;
    if (value_freq && Dv % 2) return (int)hipErrorInvalidValue;
    // A token's heads go to as many workgroups as give the step about two per compute unit (a decode step has few
    // tokens: one workgroup per token left the GPU idle), at most one per head.
    int groups = (512 + N - 1) / N;
    const int fit = (int)(((size_t)(Hq + Hkv) * D * sizeof(float) + 32 * 1024 - 1) / (32 * 1024));   // (and their heads fit LDS)
    if (groups < fit) groups = fit;
    if (groups > Hq + Hkv) groups = Hq + Hkv;
    if (groups > 65535) groups = 65535;
    const int per = (Hq + Hkv + groups - 1) / groups;
    groups = (Hq + Hkv + per - 1) / per;
    const size_t lds = (size_t)per * D * sizeof(float);
    if (lds > 60 * 1024) return (int)hipErrorInvalidValue;
#define SOC_WP(T)                                                                                                             \
    hipLaunchKernelGGL(window_prepare_kernel<T>, dim3(N, groups), dim3(256), lds, stream, (const T*)x, ld, col_q, col_k,       \
                       col_v, bias, (T*)q_out, (T*)k_pool, (T*)v_pool, table, table_width, token_rows, positions, q_gain,      \
                       k_gain, norm, eps, inv_freq, half, magnitude, value_freq, Hq, Hkv, D, Dv, P, BS, per)
    if (dtype == 0) SOC_WP(float); else SOC_WP(bf16);
#undef SOC_WP
    return soc_last_error();
}

// ---- the means of the blocks that a step completes --------------------------------------------------------------
// A sequence of the step that brings positions start .. end - 1 completes the blocks b with b * per + per - 1 among
// them: start / per <= b < end / per. Mean key and mean value of block b, over the per tokens' entries in the pools
// [pages, Hkv, BS, P] (summed in float32: every fourth position in order, then the four sums), go to entry b of the row's pages of means
// (same shape, a table of their own). grid (blocks a sequence may complete, sequences, kv heads).
template <typename T>
__global__ void __launch_bounds__(256)
pool_blocks_kernel(const T* __restrict__ k_pool, const T* __restrict__ v_pool, const int* __restrict__ table, int table_width,
                   T* __restrict__ mk_pool, T* __restrict__ mv_pool, const int* __restrict__ mtable, int mtable_width,
                   const int* __restrict__ seq_qstart, const int* __restrict__ seq_rows, const int* __restrict__ seq_ctx,
                   int Hkv, int P, int BS, int per) {
    // four waves take every fourth position of the block each; their sums meet in LDS, in the waves' order
    __shared__ float part_k[3][256], part_v[3][256];
    const int seq = blockIdx.y, kvh = blockIdx.z;
    const int n = seq_qstart[seq + 1] - seq_qstart[seq];
    const int end = seq_ctx[seq], start = end - n;
    if (n <= 0 || start < 0) return;
    const int b = start / per + blockIdx.x;
    if (b >= end / per) return;
    const int row = seq_rows[seq];
    const int* pages = table + (size_t)row * table_width;
    const int mpage = mtable[(size_t)row * mtable_width + b / BS];
    const size_t dst = (((size_t)mpage * Hkv + kvh) * BS + (size_t)(b % BS)) * P;
    const float inv = 1.f / (float)per;
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    for (int e0 = 0; e0 < P; e0 += 64) {                   // (P <= 256: the pools' head size)
        const int e = e0 + lane;
        float sk = 0.f, sv = 0.f;
        if (e < P) {
            for (int t = wave; t < per; t += 4) {
                const int pos = b * per + t;
                const size_t src = (((size_t)pages[pos / BS] * Hkv + kvh) * BS + (size_t)(pos % BS)) * P + e;
                sk += to_float(k_pool[src]);
                sv += to_float(v_pool[src]);
            }
        }
        if (wave > 0) { part_k[wave - 1][e0 + lane] = sk; part_v[wave - 1][e0 + lane] = sv; }
        __syncthreads();
        if (wave == 0 && e < P) {
#pragma unroll
            for (int w = 0; w < 3; ++w) { sk += part_k[w][e0 + lane]; sv += part_v[w][e0 + lane]; }
            mk_pool[dst + e] = from_float<T>(sk * inv);
            mv_pool[dst + e] = from_float<T>(sv * inv);
        }
    }
}

SOC_EXPORT int soc_pool_blocks(const void* k_pool, const void* v_pool, const int* table, int table_width, void* mk_pool,
                               void* mv_pool, const int* mtable, int mtable_width, const int* seq_qstart, const int* seq_rows,
                               const int* seq_ctx, int n_seqs, int max_q_len, int Hkv, int P, int BS, int per, int dtype,
                               hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (per < 1 || BS < 1 || Hkv < 1 || P < 1 || P > 256 || n_seqs > 65535 || Hkv > 65535 || max_q_len < 1) return (int)hipErrorInvalidValue;
    const dim3 grid(max_q_len / per + 1, n_seqs, Hkv);
#define SOC_PB(T)                                                                                                              \
    hipLaunchKernelGGL(pool_blocks_kernel<T>, grid, dim3(256), 0, stream, (const T*)k_pool, (const T*)v_pool, table, table_width, \
                       (T*)mk_pool, (T*)mv_pool, mtable, mtable_width, seq_qstart, seq_rows, seq_ctx, Hkv, P, BS, per)
    if (dtype == 0) SOC_PB(float); else SOC_PB(bf16);
#undef SOC_PB
    return soc_last_error();
}

// ---- a head's result turned back by the query's position, and cut to the values' size -------------------------
// o [N, H, P] -> out [N, H, Dv]; value_freq (or null: no turn): pairs (2m, 2m + 1) turned by -position * value_freq[m].
template <typename T>
__global__ void turn_back_kernel(const T* __restrict__ o, T* __restrict__ out, const int* __restrict__ positions,
                                 const float* __restrict__ value_freq, size_t total, int H, int P, int Dv) {
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const int i = (int)(e % Dv);
        const size_t nh = e / Dv;
        const T* head = o + nh * P;
        float y = to_float(head[i]);
        if (value_freq) {
            const float other = to_float(head[i ^ 1]);
            float sn, cs;
            sincosf((float)positions[nh / H] * value_freq[i >> 1], &sn, &cs);
            y = (i & 1) ? y * cs - other * sn : y * cs + other * sn;
        }
        out[e] = from_float<T>(y);
    }
}

SOC_EXPORT int soc_turn_back(const void* o, void* out, const int* positions, const float* value_freq, int N, int H, int P, int Dv,
                             int dtype, hipStream_t stream) {
    const size_t total = (size_t)N * H * Dv;
    if (!total) return 0;
    if (Dv > P || (value_freq && Dv % 2)) return (int)hipErrorInvalidValue;
    const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
    if (dtype == 0)
        hipLaunchKernelGGL(turn_back_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)o, (float*)out, positions,
                           value_freq, total, H, P, Dv);
    else
        hipLaunchKernelGGL(turn_back_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)o, (bf16*)out, positions,
                           value_freq, total, H, P, Dv);
    return soc_last_error();
}

// q (activated if act, scaled), k (activated if act) and, with z, the decay exp(logsigmoid(z + z_bias) / tau) of every
// token, head and key channel, float32: prep [N, 2 or 3, H * D]. Ahead of the walk over a long portion, where each of a
// head's workgroups would otherwise take them again.
template <typename T>
__global__ void linear_prepare_kernel(const T* __restrict__ x, int ld, int col_q, int col_k, float q_scale, int act,
                                      const float* __restrict__ z, const float* __restrict__ z_bias, float inv_tau, int HD,
                                      size_t total, float* __restrict__ prep) {
    const int planes = z ? 3 : 2;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const int c = (int)(e % HD);
        const size_t n = e / HD;
        float a = to_float(x[n * ld + col_q + c]), b = to_float(x[n * ld + col_k + c]);
        if (act) { a = cmp_silu(a); b = cmp_silu(b); }
        float* row = prep + n * planes * HD + c;
        row[0] = a * q_scale;
        row[HD] = b;
        if (z) {
            const float u = z[n * HD + c] + z_bias[c];
            row[2 * (size_t)HD] = expf((fminf(u, 0.f) - log1pf(expf(-fabsf(u)))) * inv_tau);
        }
    }
}

// ---- linear attention: S <- diag(decay) S + k v^T, o = S^T q ------------------------------------------------------
// x: rows of ld elements with H heads of D (q, from col_q; k, from col_k) and H heads of Dv (v, from col_v); with
// act they pass silu; q is scaled by q_scale. CHANNEL: the decay of token t, head h, key channel i is
// exp(logsigmoid(z[t, h D + i] + z_bias[h D + i]) / tau), z float32; else decays[h]. The state [H, D, Dv] of the
// sequence's row is float32. prepared: prep [N, 3, H D] (q, k, decay per token, head and key channel, float32) comes
// filled from the caller and nothing else of q and k is read. ones: the last ``ones`` of the Dv value columns are
// not in x (whose heads hold Dv - ones) and read 1. A workgroup owns CW columns of one head, thread (part, column) a slice of the keys;
// tokens go in batches staged through LDS with the next batch's loads in flight. o: float32 [N, H * Dv].
template <typename T, int DK, int CW, bool CHANNEL>
__global__ void __launch_bounds__(256)
linear_attention_kernel(const T* __restrict__ x, int ld, int col_q, int col_k, int col_v, float q_scale, int act,
                        const float* __restrict__ decays, const float* __restrict__ z, const float* __restrict__ z_bias,
                        float inv_tau, int H, int D, int Dv, float* __restrict__ state, size_t stride, int offset,
                        const int* __restrict__ seq_qstart, const int* __restrict__ seq_rows, const float* __restrict__ prep,
                        int ones, float* __restrict__ out) {
    constexpr int REC_TB = rec_batch(DK), PARTS = 256 / CW, KPT = DK / PARTS, STAGE = (REC_TB * DK + 255) / 256;
    __shared__ float sq[2][REC_TB][DK], sk[2][REC_TB][DK];
    __shared__ float sa[CHANNEL ? 2 : 1][CHANNEL ? REC_TB : 1][CHANNEL ? DK : 1];
    __shared__ float red[REC_TB][PARTS][CW];
    const int blocks = (Dv + CW - 1) / CW;
    const int head = blockIdx.x / blocks, seq = blockIdx.y, tid = threadIdx.x;
    const int lo = seq_qstart[seq], hi = seq_qstart[seq + 1];
    if (lo >= hi) return;
    const int col0 = (blockIdx.x % blocks) * CW;
    const int col = col0 + tid % CW, part = tid / CW, i0 = part * KPT;
    const bool live = col < Dv;
    float* S = state + (size_t)seq_rows[seq] * stride + offset + (size_t)head * D * Dv;
    const float decay = CHANNEL ? 0.f : decays[head];
    float s[KPT];
#pragma unroll
    for (int ii = 0; ii < KPT; ++ii) s[ii] = (live && i0 + ii < D) ? S[(size_t)(i0 + ii) * Dv + col] : 0.f;

    float fq[STAGE], fk[STAGE], fa[CHANNEL ? STAGE : 1], fv[REC_TB];
    auto fetch = [&](int n0) {
#pragma unroll
        for (int q = 0; q < STAGE; ++q) {
            const int e = tid + q * 256, t = e / DK, i = e % DK;
            const bool in = t < REC_TB && n0 + t < hi && i < D;
            float a = 0.f, b = 0.f, c = 1.f;
            if (in && prep) {                          // activated, scaled and the decay taken ahead of the walk
                const size_t HD = (size_t)H * D;
                const float* row = prep + (size_t)(n0 + t) * (CHANNEL ? 3 : 2) * HD + head * D + i;
                a = row[0];
                b = row[HD];
                if (CHANNEL) c = row[2 * HD];
            } else if (in) {
                const T* row = x + (size_t)(n0 + t) * ld + head * D + i;
                a = to_float(row[col_q]);
                b = to_float(row[col_k]);
                if (act) { a = cmp_silu(a); b = cmp_silu(b); }
                a *= q_scale;
                if (CHANNEL) {
                    const float u = z[(size_t)(n0 + t) * H * D + head * D + i] + z_bias[head * D + i];
                    // log(sigmoid(u)) = min(u, 0) - log(1 + exp(-|u|))
                    c = expf((fminf(u, 0.f) - log1pf(expf(-fabsf(u)))) * inv_tau);
                }
            }
            fq[q] = a;
            fk[q] = b;
            if (CHANNEL) fa[q] = c;
        }
#pragma unroll
        for (int t = 0; t < REC_TB; ++t) {
            const int held = Dv - ones;
            float v = (live && n0 + t < hi) ? (col < held ? to_float(x[(size_t)(n0 + t) * ld + col_v + head * held + col]) : 1.f) : 0.f;
            fv[t] = act ? cmp_silu(v) : v;
        }
    };
    auto land = [&](int buf) {
#pragma unroll
        for (int q = 0; q < STAGE; ++q) {
            const int e = tid + q * 256, t = e / DK, i = e % DK;
            if (t < REC_TB) {
                sq[buf][t][i] = fq[q];
                sk[buf][t][i] = fk[q];
                if (CHANNEL) sa[buf][t][i] = fa[q];
            }
        }
    };
    fetch(lo);
    land(0);
    lds_barrier();
    int buf = 0;
    for (int n0 = lo; n0 < hi; n0 += REC_TB, buf ^= 1) {
        const int nb = min(REC_TB, hi - n0);
        const bool more = n0 + REC_TB < hi;
        float vj[REC_TB];
#pragma unroll
        for (int t = 0; t < REC_TB; ++t) vj[t] = fv[t];
        if (more) fetch(n0 + REC_TB);
#pragma unroll
        for (int t = 0; t < REC_TB; ++t) {
            if (t < nb) {
                float acc = 0.f;
#pragma unroll
                for (int ii = 0; ii < KPT; ++ii) {
                    const float dec = CHANNEL ? sa[CHANNEL ? buf : 0][CHANNEL ? t : 0][CHANNEL ? i0 + ii : 0] : decay;
                    s[ii] = fmaf(dec, s[ii], sk[buf][t][i0 + ii] * vj[t]);
                    acc = fmaf(sq[buf][t][i0 + ii], s[ii], acc);
                }
                red[t][part][tid % CW] = acc;
            }
        }
        lds_barrier();
        for (int f = tid; f < REC_TB * CW; f += 256) {
            const int t = f / CW, cl = f % CW;
            if (t < nb && col0 + cl < Dv) {
                float o = 0.f;
#pragma unroll
                for (int pp = 0; pp < PARTS; ++pp) o += red[t][pp][cl];
                out[(size_t)(n0 + t) * H * Dv + (size_t)head * Dv + col0 + cl] = o;
            }
        }
        if (more) land(buf ^ 1);
        lds_barrier();
    }
    if (live) {
#pragma unroll
        for (int ii = 0; ii < KPT; ++ii)
            if (i0 + ii < D) S[(size_t)(i0 + ii) * Dv + col] = s[ii];
    }
}

template <typename T, int DK>
static void launch_linear_attention(const void* x, int ld, int col_q, int col_k, int col_v, float q_scale, int act,
                                    const float* decays, const float* z, const float* z_bias, float inv_tau, int H, int D, int Dv,
                                    float* state, long long stride, int offset, const int* seq_qstart, const int* seq_rows,
                                    const float* prep, int prepared, int ones, float* out, int n_seqs, int cw, hipStream_t stream) {
#define SOC_LA_LAUNCH(CW, CH)                                                                                                  \
    hipLaunchKernelGGL((linear_attention_kernel<T, DK, CW, CH>), dim3(H * ((Dv + CW - 1) / CW), n_seqs), dim3(256), 0, stream, \
                       (const T*)x, ld, col_q, col_k, col_v, q_scale, act, decays, z, z_bias, inv_tau, H, D, Dv, state,        \
                       (size_t)stride, offset, seq_qstart, seq_rows, prep, ones, out)
    if (z || prepared) { if (cw == 16) SOC_LA_LAUNCH(16, true); else SOC_LA_LAUNCH(64, true); }
    else   { if (cw == 16) SOC_LA_LAUNCH(16, false); else SOC_LA_LAUNCH(64, false); }
#undef SOC_LA_LAUNCH
}

SOC_EXPORT int soc_linear_attention(const void* x, int ld, int col_q, int col_k, int col_v, float q_scale, int act,
                                    const float* decays, const float* z, const float* z_bias, float tau, int H, int D, int Dv,
                                    float* state, long long stride, int offset, const int* seq_qstart, const int* seq_rows,
                                    float* prep, int prepared, int ones, int n_tokens, float* out, int n_seqs, int max_q_len,
                                    int dtype, hipStream_t stream) {
    if (n_seqs <= 0 || H <= 0) return 0;
    if (D < 1 || D > 256 || Dv < 1 || n_seqs > 65535 || ones < 0 || ones >= Dv) return (int)hipErrorInvalidValue;
    if (prepared ? (!prep || z || decays)
                 : ((z == nullptr) == (decays == nullptr) || (z && (!z_bias || !(tau > 0.f))))) return (int)hipErrorInvalidValue;
    const int cw = columns_per_workgroup(H, Dv, n_seqs, max_q_len);
    const float inv_tau = z ? 1.f / tau : 0.f;
    if (prep && !prepared) {                                            // scratch [n_tokens, 2 or 3, H * D]
        if (n_tokens <= 0) return (int)hipErrorInvalidValue;
        const size_t total = (size_t)n_tokens * H * D;
        const int blocks = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
        if (dtype == 0)
            hipLaunchKernelGGL(linear_prepare_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)x, ld, col_q, col_k,
                               q_scale, act, z, z_bias, inv_tau, H * D, total, prep);
        else
            hipLaunchKernelGGL(linear_prepare_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)x, ld, col_q, col_k,
                               q_scale, act, z, z_bias, inv_tau, H * D, total, prep);
    }
#define SOC_LA_F32(DK) launch_linear_attention<float, DK>(x, ld, col_q, col_k, col_v, q_scale, act, decays, z, z_bias, inv_tau, H, D, Dv, state, stride, offset, seq_qstart, seq_rows, prep, prepared, ones, out, n_seqs, cw, stream)
#define SOC_LA_BF16(DK) launch_linear_attention<bf16, DK>(x, ld, col_q, col_k, col_v, q_scale, act, decays, z, z_bias, inv_tau, H, D, Dv, state, stride, offset, seq_qstart, seq_rows, prep, prepared, ones, out, n_seqs, cw, stream)
    if (dtype == 0) { SOC_BY_STATE_SIZE(D, SOC_LA_F32) } else { SOC_BY_STATE_SIZE(D, SOC_LA_BF16) }
    return soc_last_error();
}

// ---- a_scale * (a + bias) + b_scale * b, float32 ------------------------------------------------------------------
// a, b [N, d]: float32 or the compute dtype each (b may be null); bias float32 [d] or null; out float32 [N, d].
template <typename T>
__global__ void scaled_sum_kernel(const void* __restrict__ a, int a_f32, float a_scale, const void* __restrict__ b, int b_f32,
                                  float b_scale, const float* __restrict__ bias, float* __restrict__ out, size_t total, int d) {
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        float y = a_f32 ? ((const float*)a)[e] : to_float(((const T*)a)[e]);
        if (bias) y += bias[e % d];
        y *= a_scale;
        if (b) y = fmaf(b_scale, b_f32 ? ((const float*)b)[e] : to_float(((const T*)b)[e]), y);
        out[e] = y;
    }
}

SOC_EXPORT int soc_scaled_sum(const void* a, int a_f32, float a_scale, const void* b, int b_f32, float b_scale, const float* bias,
                              float* out, int N, int d, int dtype, hipStream_t stream) {
    const size_t total = (size_t)N * d;
    if (!total) return 0;
    const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
    if (dtype == 0)
        hipLaunchKernelGGL(scaled_sum_kernel<float>, dim3(blocks), dim3(256), 0, stream, a, 1, a_scale, b, 1, b_scale, bias, out, total, d);
    else
        hipLaunchKernelGGL(scaled_sum_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, a, a_f32, a_scale, b, b_f32, b_scale, bias, out, total, d);
    return soc_last_error();
}

// ---- gelu_tanh(gate) * up -------------------------------------------------------------------------------------------
// gate_up: rows of ld elements, gate in the first ff, up in the next ff; out [N, ff].
template <typename T>
__global__ void glu_gelu_kernel(const T* __restrict__ gate_up, T* __restrict__ out, size_t total, int ff, int ld) {
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const size_t n = e / ff;
        const int c = (int)(e % ff);
        const float g = to_float(gate_up[n * ld + c]), u = to_float(gate_up[n * ld + ff + c]);
        const float t = tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g));
        out[e] = from_float<T>(0.5f * g * (1.f + t) * u);
    }
}

SOC_EXPORT int soc_glu_gelu(const void* gate_up, void* out, int N, int ff, int ld, int dtype, hipStream_t stream) {
    const size_t total = (size_t)N * ff;
    if (!total) return 0;
    if (ff < 1 || 2 * ff > ld) return (int)hipErrorInvalidValue;
    const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
    if (dtype == 0)
        hipLaunchKernelGGL(glu_gelu_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)gate_up, (float*)out, total, ff, ld);
    else
        hipLaunchKernelGGL(glu_gelu_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out, total, ff, ld);
    return soc_last_error();
}
