// Kernels of the mixers beyond grouped-query attention, and of blocks with norms on both
// sides of a branch: the gated close of a branch, a clamped gated activation, the blends of
// a token with the one before it, two recurrences with a matrix state per head (decay per key
// channel; scalar decay), a short causal convolution, a gated group norm, and what attention
// over a cached latent needs around the paged-attention kernels (norm + rotation + page write
// of the latent, rotation of the queries, one small product per head).
//
// Statistics, gates, decays, exponentials, angles and states are float32 whatever the compute
// dtype; a value is rounded once, where it is stored in the compute dtype.
//
// Sequences: kernels that carry state walk the tokens of each sequence of the step in order.
// seq_qstart [S + 1] gives each sequence's tokens among the step's, seq_rows [S] its row of
// the state tensor [rows, stride] (float32).
#include "common.h"
#include "recurrent.h"

__device__ __forceinline__ float soc_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }

__device__ __forceinline__ void store8(float* p, const float (&x)[8]) {
    *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(x[4], x[5], x[6], x[7]);
}
__device__ __forceinline__ void store8(bf16* p, const float (&x)[8]) {
    *reinterpret_cast<uint4*>(p) = make_uint4(pack_bf16x2(x[0], x[1]), pack_bf16x2(x[2], x[3]), pack_bf16x2(x[4], x[5]),
                                              pack_bf16x2(x[6], x[7]));
}


// ---- the close of a branch ---------------------------------------------------------------------
// residual += mult * gain * g / rms(g) with g = y * sigmoid(logits + bias) (no gate: g = y); the logits are the
// first d elements of rows of ldg elements (they may be columns of a wider product);
// then, if next_gain is given, out = residual / rms(residual) * next_gain. y is in the compute dtype, or float32 if
// y_f32; y_bias (float32 [d], or null) is added to it first.
template <typename T>
__device__ __forceinline__ float branch_result(const void* y, int y_f32, const float* y_bias, size_t at, int c) {
    const float v = y_f32 ? ((const float*)y)[at] : to_float(((const T*)y)[at]);
    return y_bias ? v + y_bias[c] : v;
}

template <typename T>
__global__ void __launch_bounds__(256)
gated_norm_add_kernel(float* __restrict__ residual, const void* __restrict__ y, int y_f32, const float* __restrict__ y_bias,
                      const T* __restrict__ logits, int ldg,
                      const float* __restrict__ bias, const float* __restrict__ gain, float eps, float mult,
                      const float* __restrict__ next_gain, float next_eps, T* __restrict__ out, int d) {
    __shared__ float scratch[16];
    const size_t base = (size_t)blockIdx.x * d, gbase = (size_t)blockIdx.x * ldg;
    float ss = 0.f;
    for (int c = threadIdx.x; c < d; c += blockDim.x) {
        float g = branch_result<T>(y, y_f32, y_bias, base + c, c);
        if (logits) g *= soc_sigmoid(to_float(logits[gbase + c]) + bias[c]);
        ss += g * g;
    }
    ss = block_sum(ss, scratch);
    const float scale = mult / sqrtf(ss / (float)d + eps);
    float rr = 0.f;
    for (int c = threadIdx.x; c < d; c += blockDim.x) {
        float g = branch_result<T>(y, y_f32, y_bias, base + c, c);
        if (logits) g *= soc_sigmoid(to_float(logits[gbase + c]) + bias[c]);
        const float r = residual[base + c] + scale * gain[c] * g;
        residual[base + c] = r;
        rr += r * r;
    }
    if (!next_gain) return;
    rr = block_sum(rr, scratch);
    const float inv = 1.f / sqrtf(rr / (float)d + next_eps);
    for (int c = threadIdx.x; c < d; c += blockDim.x)
        out[base + c] = from_float<T>(residual[base + c] * inv * next_gain[c]);
}

// The same with the row in registers (PER elements per thread, d <= 256 * PER): every element is
// read once, all loads are issued before the first is used.
template <typename T, int PER>
__global__ void __launch_bounds__(256)
gated_norm_add_regs_kernel(float* __restrict__ residual, const void* __restrict__ y, int y_f32, const float* __restrict__ y_bias,
                           const T* __restrict__ logits, int ldg,
                           const float* __restrict__ bias, const float* __restrict__ gain, float eps, float mult,
                           const float* __restrict__ next_gain, float next_eps, T* __restrict__ out, int d) {
    __shared__ float scratch[16];
    const size_t base = (size_t)blockIdx.x * d, gbase = (size_t)blockIdx.x * ldg;
    float g[PER], res[PER], gate[PER], gn[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int c = threadIdx.x + i * 256;
        const bool in = c < d;
        g[i] = in ? branch_result<T>(y, y_f32, y_bias, base + c, c) : 0.f;
        gate[i] = (in && logits) ? to_float(logits[gbase + c]) + bias[c] : 0.f;
        res[i] = in ? residual[base + c] : 0.f;
        gn[i] = in ? gain[c] : 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        if (logits) g[i] *= soc_sigmoid(gate[i]);
        ss += g[i] * g[i];
    }
    ss = block_sum(ss, scratch);
    const float scale = mult / sqrtf(ss / (float)d + eps);
    float rr = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int c = threadIdx.x + i * 256;
        res[i] += scale * gn[i] * g[i];
        if (c < d) residual[base + c] = res[i];
        rr += res[i] * res[i];
    }
    if (!next_gain) return;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int c = threadIdx.x + i * 256;
        gn[i] = c < d ? next_gain[c] : 0.f;
    }
    rr = block_sum(rr, scratch);
    const float inv = 1.f / sqrtf(rr / (float)d + next_eps);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int c = threadIdx.x + i * 256;
        if (c < d) out[base + c] = from_float<T>(res[i] * inv * gn[i]);
    }
}

// The same again for widths that are multiples of 8, eight consecutive elements per load (16 bytes of
// bfloat16, 32 of float32), CH such pieces per thread (d <= 2048 * CH); the next norm's gain comes with
// the first loads, so the kernel waits for memory once.
template <typename T, int CH>
__global__ void __launch_bounds__(256)
gated_norm_add_vec8_kernel(float* __restrict__ residual, const void* __restrict__ y, int y_f32, const float* __restrict__ y_bias,
                           const T* __restrict__ logits, int ldg,
                           const float* __restrict__ bias, const float* __restrict__ gain, float eps, float mult,
                           const float* __restrict__ next_gain, float next_eps, T* __restrict__ out, int d) {
    __shared__ float scratch[16];
    const size_t base = (size_t)blockIdx.x * d, gbase = (size_t)blockIdx.x * ldg;
    float g[CH][8], res[CH][8], gate[CH][8], gn[CH][8], nx[CH][8];
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int c = (threadIdx.x + i * 256) * 8;
        if (c < d) {
            if (y_f32) VecLoad<float, 8>::load((const float*)y + base + c, g[i]);
            else VecLoad<T, 8>::load((const T*)y + base + c, g[i]);
            if (y_bias) {
                float yb[8];
                VecLoad<float, 8>::load(y_bias + c, yb);
#pragma unroll
                for (int e = 0; e < 8; ++e) g[i][e] += yb[e];
            }
            VecLoad<float, 8>::load(residual + base + c, res[i]);
            VecLoad<float, 8>::load(gain + c, gn[i]);
            if (logits) {
                float b[8];
                VecLoad<T, 8>::load(logits + gbase + c, gate[i]);
                VecLoad<float, 8>::load(bias + c, b);
#pragma unroll
                for (int e = 0; e < 8; ++e) gate[i][e] += b[e];
            }
            if (next_gain) VecLoad<float, 8>::load(next_gain + c, nx[i]);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) g[i][e] = res[i][e] = gn[i][e] = gate[i][e] = nx[i][e] = 0.f;
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < CH; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (logits) g[i][e] *= soc_sigmoid(gate[i][e]);
            ss += g[i][e] * g[i][e];
        }
    ss = block_sum(ss, scratch);
    const float scale = mult / sqrtf(ss / (float)d + eps);
    float rr = 0.f;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int c = (threadIdx.x + i * 256) * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            res[i][e] += scale * gn[i][e] * g[i][e];
            rr += res[i][e] * res[i][e];
        }
        if (c < d) store8(residual + base + c, res[i]);
    }
    if (!next_gain) return;
    rr = block_sum(rr, scratch);
    const float inv = 1.f / sqrtf(rr / (float)d + next_eps);
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int c = (threadIdx.x + i * 256) * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) res[i][e] *= inv * nx[i][e];
        if (c < d) store8(out + base + c, res[i]);
    }
}

template <typename T>
static void launch_gated_norm_add(float* residual, const void* y, int y_f32, const float* y_bias, const void* logits, int ldg, const float* bias, const float* gain,
                                  float eps, float mult, const float* next_gain, float next_eps, void* out, int N, int d,
                                  hipStream_t stream) {
#define SOC_GNA(PER)                                                                                                    \
    hipLaunchKernelGGL((gated_norm_add_regs_kernel<T, PER>), dim3(N), dim3(256), 0, stream, residual, y, y_f32, y_bias, \
                       (const T*)logits, ldg, bias, gain, eps, mult, next_gain, next_eps, (T*)out, d)
#define SOC_GNA8(CH)                                                                                                    \
    hipLaunchKernelGGL((gated_norm_add_vec8_kernel<T, CH>), dim3(N), dim3(256), 0, stream, residual, y, y_f32, y_bias,  \
                       (const T*)logits, ldg, bias, gain, eps, mult, next_gain, next_eps, (T*)out, d)
    // (pieces of eight elements: the width, the logits' rows and their first element all sit at multiples of 8)
    const bool by8 = d % 8 == 0 && ldg % 8 == 0 && ((uintptr_t)logits % (8 * sizeof(T))) == 0 &&
                     ((uintptr_t)y % (y_f32 ? 32 : 8 * sizeof(T))) == 0;
    if (by8 && d <= 2048) SOC_GNA8(1);
    else if (by8 && d <= 4096) SOC_GNA8(2);
    else if (by8 && d <= 8192) SOC_GNA8(4);
    else if (d <= 1024) SOC_GNA(4);
    else if (d <= 2048) SOC_GNA(8);
    else if (d <= 4096) SOC_GNA(16);
    else if (d <= 8192) SOC_GNA(32);
    else
        hipLaunchKernelGGL(gated_norm_add_kernel<T>, dim3(N), dim3(256), 0, stream, residual, y, y_f32, y_bias, (const T*)logits,
                           ldg, bias, gain, eps, mult, next_gain, next_eps, (T*)out, d);
}

SOC_EXPORT int soc_gated_norm_add(float* residual, const void* y, int y_f32, const float* y_bias, const void* logits, int ldg, const float* bias,
                                  const float* gain, float eps, float mult, const float* next_gain, float next_eps,
                                  void* out, int N, int d, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (dtype == 0) launch_gated_norm_add<float>(residual, y, y_f32, y_bias, logits, ldg, bias, gain, eps, mult, next_gain, next_eps, out, N, d, stream);
    else launch_gated_norm_add<bf16>(residual, y, y_f32, y_bias, logits, ldg, bias, gain, eps, mult, next_gain, next_eps, out, N, d, stream);
    return soc_last_error();
}

// ---- g * sigmoid(slope g) * (u + 1), g = min(gate, limit), u = clamp(up, -limit, limit) ---------
// gate and up are the first 2 ff elements of rows of ld elements.
template <typename T>
__global__ void glu_clamped_kernel(const T* __restrict__ gate_up, T* __restrict__ out, size_t total, int ff, int ld,
                                   float limit, float slope) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t n = i / ff, c = i % ff;
    const float g = fminf(to_float(gate_up[n * ld + c]), limit);
    const float u = fminf(fmaxf(to_float(gate_up[n * ld + ff + c]), -limit), limit);
    out[i] = from_float<T>(g * soc_sigmoid(slope * g) * (u + 1.f));
}

// (eight consecutive elements per lane where ff is a multiple of 8)
template <typename T>
__global__ void glu_clamped_vec8_kernel(const T* __restrict__ gate_up, T* __restrict__ out, size_t groups, int ff, int ld,
                                        float limit, float slope) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= groups) return;
    const int per_row = ff / 8;
    const size_t n = i / per_row, c = (i % per_row) * 8;
    float g[8], u[8], y[8];
    VecLoad<T, 8>::load(gate_up + n * ld + c, g);
    VecLoad<T, 8>::load(gate_up + n * ld + ff + c, u);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float gg = fminf(g[e], limit), uu = fminf(fmaxf(u[e], -limit), limit);
        y[e] = gg * soc_sigmoid(slope * gg) * (uu + 1.f);
    }
    store8(out + n * ff + c, y);
}

SOC_EXPORT int soc_glu_clamped(const void* gate_up, void* out, int N, int ff, int ld, float limit, float slope, int dtype,
                               hipStream_t stream) {
    const size_t total = (size_t)N * ff;
    if (total == 0) return 0;
    if (ld < 2 * ff) return (int)hipErrorInvalidValue;
    if (ff % 8 == 0 && ld % 8 == 0) {
        const size_t groups = total / 8;
        const dim3 grid((unsigned)((groups + 255) / 256));
        if (dtype == 0)
            hipLaunchKernelGGL(glu_clamped_vec8_kernel<float>, grid, dim3(256), 0, stream, (const float*)gate_up, (float*)out,
                               groups, ff, ld, limit, slope);
        else
            hipLaunchKernelGGL(glu_clamped_vec8_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out,
                               groups, ff, ld, limit, slope);
        return soc_last_error();
    }
    const dim3 grid((unsigned)((total + 255) / 256));
    if (dtype == 0)
        hipLaunchKernelGGL(glu_clamped_kernel<float>, grid, dim3(256), 0, stream, (const float*)gate_up, (float*)out,
                           total, ff, ld, limit, slope);
    else
        hipLaunchKernelGGL(glu_clamped_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out,
                           total, ff, ld, limit, slope);
    return soc_last_error();
}

// ---- blends of a token's input with the one before it ---------------------------------------------
// out[s, n, c] = h[n, c] + (prev[n, c] - h[n, c]) * mu[s, c]; prev of a sequence's first token of
// the step is what the row's state holds, which then becomes the input of its last token. Grid
// (chunks of SHIFT_CHUNK tokens, sequences, blocks of 256 columns): the workgroups of a sequence's
// first chunk are the only ones that touch the state, each thread its own column, reading before writing.
constexpr int SHIFT_CHUNK = 8;

template <typename T>
__global__ void __launch_bounds__(256)
token_shift_kernel(const T* __restrict__ h, const float* __restrict__ mu, int n_streams, float* __restrict__ state,
                   size_t stride, int offset, const int* __restrict__ seq_qstart, const int* __restrict__ seq_rows,
                   T* __restrict__ out, int N, int d) {
    const int seq = blockIdx.y;
    const int lo = seq_qstart[seq], hi = seq_qstart[seq + 1];
    const int first = lo + blockIdx.x * SHIFT_CHUNK;
    if (first >= hi) return;
    const int last = min(first + SHIFT_CHUNK, hi);
    float* kept = state + (size_t)seq_rows[seq] * stride + offset;
    const int c = blockIdx.z * blockDim.x + threadIdx.x;
    if (c < d) {
        float prev = first == lo ? kept[c] : to_float(h[(size_t)(first - 1) * d + c]);
        for (int n = first; n < last; ++n) {
            const float cur = to_float(h[(size_t)n * d + c]);
            const float diff = prev - cur;
            for (int s = 0; s < n_streams; ++s)
                out[((size_t)s * N + n) * d + c] = from_float<T>(cur + diff * mu[(size_t)s * d + c]);
            prev = cur;
        }
        if (first == lo) kept[c] = to_float(h[(size_t)(hi - 1) * d + c]);
    }
}

SOC_EXPORT int soc_token_shift(const void* h, const float* mu, int n_streams, float* state, long long stride, int offset,
                               const int* seq_qstart, const int* seq_rows, void* out, int N, int d, int n_seqs,
                               int max_q_len, int dtype, hipStream_t stream) {
    if (N <= 0 || n_seqs <= 0) return 0;
    if (n_seqs > 65535 || (d + 255) / 256 > 65535) return (int)hipErrorInvalidValue;
    const dim3 grid((max_q_len + SHIFT_CHUNK - 1) / SHIFT_CHUNK, n_seqs, (d + 255) / 256);
    if (dtype == 0)
        hipLaunchKernelGGL(token_shift_kernel<float>, grid, dim3(256), 0, stream, (const float*)h, mu, n_streams, state,
                           (size_t)stride, offset, seq_qstart, seq_rows, (float*)out, N, d);
    else
        hipLaunchKernelGGL(token_shift_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)h, mu, n_streams, state,
                           (size_t)stride, offset, seq_qstart, seq_rows, (bf16*)out, N, d);
    return soc_last_error();
}

// ---- decay = exp(-exp(tanh(t) W2^T + w0)) --------------------------------------------------------
// t [N, rank] float32; W2 transposed, [rank, C] (consecutive threads read consecutive elements); grid (blocks
// of 256 channels, tokens), a thread per channel, tanh(t) of the token in LDS.
template <typename T>
__global__ void __launch_bounds__(256)
wkv_decay_kernel(const float* __restrict__ t, const T* __restrict__ w2, const float* __restrict__ w0,
                 float* __restrict__ out, int C, int rank) {
    extern __shared__ float th[];
    const int n = blockIdx.y;
    for (int j = threadIdx.x; j < rank; j += blockDim.x) th[j] = tanhf(t[(size_t)n * rank + j]);
    __syncthreads();
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c < C) {
        float z = 0.f;
        for (int j = 0; j < rank; ++j) z = fmaf(th[j], to_float(w2[(size_t)j * C + c]), z);
        out[(size_t)n * C + c] = expf(-expf(z + w0[c]));
    }
}

SOC_EXPORT int soc_wkv_decay(const float* t, const void* w2, const float* w0, float* out, int N, int C, int rank,
                             int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (N > 65535) return (int)hipErrorInvalidValue;
    const size_t lds = (size_t)rank * sizeof(float);
    if (dtype == 0)
        hipLaunchKernelGGL(wkv_decay_kernel<float>, dim3((C + 255) / 256, N), dim3(256), lds, stream, t, (const float*)w2, w0, out, C, rank);
    else
        hipLaunchKernelGGL(wkv_decay_kernel<bf16>, dim3((C + 255) / 256, N), dim3(256), lds, stream, t, (const bf16*)w2, w0, out, C, rank);
    return soc_last_error();
}

// ---- the two recurrences with a matrix state per head ---------------------------------------------------
// A workgroup of 256 threads owns CW columns of one head's state S [keys, columns] for one sequence, in
// registers: thread (part, column) holds keys part * KPT .. (part + 1) * KPT - 1 of its column (PARTS * CW =
// 256; consecutive lanes are consecutive columns). Columns never meet in the recurrence, so a head is
// spread over as many workgroups as fill the GPU (CW = 16 when sequences and heads alone give too few,
// else 64). Tokens go in batches: what all threads need of a batch (per key: r, k, decay; or B,
// C) is staged through LDS; the next batch's global loads are issued before the current batch is computed
// and land in LDS after it; the partial sums of a column's PARTS threads meet in LDS once per batch.
// Decay per key channel: o_t[j] = sum_i r_t[i] (S[i, j] + u[i] k_t[i] v_t[j]); S[i, j] <- w_t[i] S[i, j] +
// k_t[i] v_t[j]. o goes out in float32; its norm over the head is another kernel's.
template <typename T, int DK, int CW>
__global__ void __launch_bounds__(256)
wkv_kernel(const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v, const float* __restrict__ decay,
           const float* __restrict__ bonus, int H, int D, float* __restrict__ state, size_t stride, int offset,
           const int* __restrict__ seq_qstart, const int* __restrict__ seq_rows, float* __restrict__ out) {
    constexpr int REC_TB = rec_batch(DK), PARTS = 256 / CW, KPT = DK / PARTS, STAGE = (REC_TB * DK + 255) / 256;
    __shared__ float sr[2][REC_TB][DK], sk[2][REC_TB][DK], sw[2][REC_TB][DK];
    __shared__ float red[REC_TB][PARTS][CW], su[DK];
    const int blocks = (D + CW - 1) / CW;
    const int head = blockIdx.x / blocks, seq = blockIdx.y, tid = threadIdx.x;
    const int lo = seq_qstart[seq], hi = seq_qstart[seq + 1];
    if (lo >= hi) return;
    const int col0 = (blockIdx.x % blocks) * CW;
    const int col = col0 + tid % CW, part = tid / CW, i0 = part * KPT;
    const bool live = col < D;
    float* S = state + (size_t)seq_rows[seq] * stride + offset + (size_t)head * D * D;
    const size_t C = (size_t)H * D, hoff = (size_t)head * D;
    float s[KPT];
#pragma unroll
    for (int ii = 0; ii < KPT; ++ii) s[ii] = (live && i0 + ii < D) ? S[(size_t)(i0 + ii) * D + col] : 0.f;
    for (int i = tid; i < DK; i += 256) su[i] = i < D ? bonus[head * D + i] : 0.f;

    float fr[STAGE], fk[STAGE], fw[STAGE], fv[REC_TB];
    auto fetch = [&](int n0) {
#pragma unroll
        for (int q = 0; q < STAGE; ++q) {
            const int e = tid + q * 256, t = e / DK, i = e % DK;
            const bool in = t < REC_TB && n0 + t < hi && i < D;
            const size_t at = (size_t)(n0 + t) * C + hoff + i;
            fr[q] = in ? to_float(r[at]) : 0.f;
            fk[q] = in ? to_float(k[at]) : 0.f;
            fw[q] = in ? decay[at] : 0.f;
        }
#pragma unroll
        for (int t = 0; t < REC_TB; ++t)
            fv[t] = (live && n0 + t < hi) ? to_float(v[(size_t)(n0 + t) * C + hoff + col]) : 0.f;
    };
    auto land = [&](int buf) {
#pragma unroll
        for (int q = 0; q < STAGE; ++q) {
            const int e = tid + q * 256, t = e / DK, i = e % DK;
            if (t < REC_TB) { sr[buf][t][i] = fr[q]; sk[buf][t][i] = fk[q]; sw[buf][t][i] = fw[q]; }
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
                    const float kv = sk[buf][t][i0 + ii] * vj[t];
                    acc = fmaf(sr[buf][t][i0 + ii], fmaf(su[i0 + ii], kv, s[ii]), acc);
                    s[ii] = fmaf(sw[buf][t][i0 + ii], s[ii], kv);
                }
                red[t][part][tid % CW] = acc;
            }
        }
        lds_barrier();
        for (int f = tid; f < REC_TB * CW; f += 256) {
            const int t = f / CW, cl = f % CW;
            if (t < nb && col0 + cl < D) {
                float o = 0.f;
#pragma unroll
                for (int pp = 0; pp < PARTS; ++pp) o += red[t][pp][cl];
                out[(size_t)(n0 + t) * C + hoff + col0 + cl] = o;
            }
        }
        if (more) land(buf ^ 1);
        lds_barrier();
    }
    if (live) {
#pragma unroll
        for (int ii = 0; ii < KPT; ++ii)
            if (i0 + ii < D) S[(size_t)(i0 + ii) * D + col] = s[ii];
    }
}

template <typename T, int DK>
static void launch_wkv(const void* r, const void* k, const void* v, const float* decay, const float* bonus, int H, int D,
                       float* state, long long stride, int offset, const int* seq_qstart, const int* seq_rows, float* out,
                       int n_seqs, int cw, hipStream_t stream) {
#define SOC_WKV_LAUNCH(CW)                                                                                                  \
    hipLaunchKernelGGL((wkv_kernel<T, DK, CW>), dim3(H * ((D + CW - 1) / CW), n_seqs), dim3(256), 0, stream, (const T*)r, \
                       (const T*)k, (const T*)v, decay, bonus, H, D, state, (size_t)stride, offset, seq_qstart, seq_rows, out)
    if (cw == 16) SOC_WKV_LAUNCH(16); else SOC_WKV_LAUNCH(64);
}

SOC_EXPORT int soc_wkv(const void* r, const void* k, const void* v, const float* decay, const float* bonus, int H, int D,
                       float* state, long long stride, int offset, const int* seq_qstart, const int* seq_rows, float* out,
                       int n_seqs, int max_q_len, int dtype, hipStream_t stream) {
    if (n_seqs <= 0 || H <= 0) return 0;
    if (D < 1 || D > 256 || n_seqs > 65535) return (int)hipErrorInvalidValue;
    const int cw = columns_per_workgroup(H, D, n_seqs, max_q_len);
#define SOC_WKV_F32(DK) launch_wkv<float, DK>(r, k, v, decay, bonus, H, D, state, stride, offset, seq_qstart, seq_rows, out, n_seqs, cw, stream)
#define SOC_WKV_BF16(DK) launch_wkv<bf16, DK>(r, k, v, decay, bonus, H, D, state, stride, offset, seq_qstart, seq_rows, out, n_seqs, cw, stream)
    if (dtype == 0) { SOC_BY_STATE_SIZE(D, SOC_WKV_F32) } else { SOC_BY_STATE_SIZE(D, SOC_WKV_BF16) }
    return soc_last_error();
}

// Scalar decay per head: xbc [N, x (H P) | B (G Ns) | C (G Ns)]; dt = softplus(dt_raw + bias);
// S[i, p] <- exp(-exp(a_log) dt) S[i, p] + dt B[i] x[p]; y[p] = sum_i C[i] S[i, p] + skip x[p], float32.
template <typename T, int NK, int CW>
__global__ void __launch_bounds__(256)
ssd_kernel(const T* __restrict__ xbc, const float* __restrict__ dt_raw, const float* __restrict__ dt_bias,
           const float* __restrict__ a_log, const float* __restrict__ skip, int H, int P, int Ns, int G,
           float* __restrict__ state, size_t stride, int offset, const int* __restrict__ seq_qstart,
           const int* __restrict__ seq_rows, float* __restrict__ out) {
    constexpr int REC_TB = rec_batch(NK), PARTS = 256 / CW, KPT = NK / PARTS, STAGE = (REC_TB * NK + 255) / 256;
    __shared__ float sb[2][REC_TB][NK], sc[2][REC_TB][NK], skeep[2][REC_TB], sdt[2][REC_TB];
    __shared__ float red[REC_TB][PARTS][CW];
    const int blocks = (P + CW - 1) / CW;
    const int head = blockIdx.x / blocks, seq = blockIdx.y, tid = threadIdx.x;
    const int lo = seq_qstart[seq], hi = seq_qstart[seq + 1];
    if (lo >= hi) return;
    const int col0 = (blockIdx.x % blocks) * CW;
    const int col = col0 + tid % CW, part = tid / CW, i0 = part * KPT;
    const bool live = col < P;
    const int group = head / (H / G);
    const int inner = H * P, ld = inner + 2 * G * Ns;
    const int boff = inner + group * Ns, coff = inner + G * Ns + group * Ns;
    float* S = state + (size_t)seq_rows[seq] * stride + offset + (size_t)head * Ns * P;
    float s[KPT];
#pragma unroll
    for (int ii = 0; ii < KPT; ++ii) s[ii] = (live && i0 + ii < Ns) ? S[(size_t)(i0 + ii) * P + col] : 0.f;
    const float rate = expf(a_log[head]), through = skip[head], shift = dt_bias[head];
    auto step_size = [&](int n) {
        const float z = dt_raw[(size_t)n * H + head] + shift;
        return z > 20.f ? z : log1pf(expf(z));
    };

    // (a token's step size and decay are computed once, by one thread, and go through LDS with B and C)
    float fb[STAGE], fc[STAGE], fx[REC_TB], fdt = 0.f, fkeep = 1.f;
    auto fetch = [&](int n0) {
#pragma unroll
        for (int t = 0; t < REC_TB; ++t)
            fx[t] = (live && n0 + t < hi) ? to_float(xbc[(size_t)(n0 + t) * ld + head * P + col]) : 0.f;
#pragma unroll
        for (int q = 0; q < STAGE; ++q) {
            const int e = tid + q * 256, t = e / NK, i = e % NK;
            const bool in = t < REC_TB && n0 + t < hi && i < Ns;
            const T* row = xbc + (size_t)(n0 + t) * ld;
            fb[q] = in ? to_float(row[boff + i]) : 0.f;
            fc[q] = in ? to_float(row[coff + i]) : 0.f;
        }
        if (tid < REC_TB) {
            fdt = n0 + tid < hi ? step_size(n0 + tid) : 0.f;
            fkeep = expf(-rate * fdt);
        }
    };
    auto land = [&](int buf) {
#pragma unroll
        for (int q = 0; q < STAGE; ++q) {
            const int e = tid + q * 256, t = e / NK, i = e % NK;
            if (t < REC_TB) { sb[buf][t][i] = fb[q]; sc[buf][t][i] = fc[q]; }
        }
        if (tid < REC_TB) { sdt[buf][tid] = fdt; skeep[buf][tid] = fkeep; }
    };
    fetch(lo);
    land(0);
    lds_barrier();
    int buf = 0;
    for (int n0 = lo; n0 < hi; n0 += REC_TB, buf ^= 1) {
        const int nb = min(REC_TB, hi - n0);
        const bool more = n0 + REC_TB < hi;
        float xj[REC_TB];
#pragma unroll
        for (int t = 0; t < REC_TB; ++t) xj[t] = fx[t];
        if (more) fetch(n0 + REC_TB);
#pragma unroll
        for (int t = 0; t < REC_TB; ++t) {
            if (t < nb) {
                const float keep = skeep[buf][t], dx = sdt[buf][t] * xj[t];
                float acc = part == 0 ? through * xj[t] : 0.f;
#pragma unroll
                for (int ii = 0; ii < KPT; ++ii) {
                    s[ii] = fmaf(keep, s[ii], sb[buf][t][i0 + ii] * dx);
                    acc = fmaf(sc[buf][t][i0 + ii], s[ii], acc);
                }
                red[t][part][tid % CW] = acc;
            }
        }
        lds_barrier();
        for (int f = tid; f < REC_TB * CW; f += 256) {
            const int t = f / CW, cl = f % CW;
            if (t < nb && col0 + cl < P) {
                float y = 0.f;
#pragma unroll
                for (int pp = 0; pp < PARTS; ++pp) y += red[t][pp][cl];
                out[(size_t)(n0 + t) * inner + head * P + col0 + cl] = y;
            }
        }
        if (more) land(buf ^ 1);
        lds_barrier();
    }
    if (live) {
#pragma unroll
        for (int ii = 0; ii < KPT; ++ii)
            if (i0 + ii < Ns) S[(size_t)(i0 + ii) * P + col] = s[ii];
    }
}

template <typename T, int NK>
static void launch_ssd(const void* xbc, const float* dt_raw, const float* dt_bias, const float* a_log, const float* skip,
                       int H, int P, int Ns, int G, float* state, long long stride, int offset, const int* seq_qstart,
                       const int* seq_rows, float* out, int n_seqs, int cw, hipStream_t stream) {
#define SOC_SSD_LAUNCH(CW)                                                                                                   \
    hipLaunchKernelGGL((ssd_kernel<T, NK, CW>), dim3(H * ((P + CW - 1) / CW), n_seqs), dim3(256), 0, stream, (const T*)xbc, \
                       dt_raw, dt_bias, a_log, skip, H, P, Ns, G, state, (size_t)stride, offset, seq_qstart, seq_rows, out)
    if (cw == 16) SOC_SSD_LAUNCH(16); else SOC_SSD_LAUNCH(64);
}

SOC_EXPORT int soc_ssd(const void* xbc, const float* dt_raw, const float* dt_bias, const float* a_log, const float* skip,
                       int H, int P, int Ns, int G, float* state, long long stride, int offset, const int* seq_qstart,
                       const int* seq_rows, float* out, int n_seqs, int max_q_len, int dtype, hipStream_t stream) {
    if (n_seqs <= 0 || H <= 0) return 0;
    if (Ns < 1 || Ns > 256 || P < 1 || G < 1 || H % G || n_seqs > 65535) return (int)hipErrorInvalidValue;
    const int cw = columns_per_workgroup(H, P, n_seqs, max_q_len);
#define SOC_SSD_F32(NK) launch_ssd<float, NK>(xbc, dt_raw, dt_bias, a_log, skip, H, P, Ns, G, state, stride, offset, seq_qstart, seq_rows, out, n_seqs, cw, stream)
#define SOC_SSD_BF16(NK) launch_ssd<bf16, NK>(xbc, dt_raw, dt_bias, a_log, skip, H, P, Ns, G, state, stride, offset, seq_qstart, seq_rows, out, n_seqs, cw, stream)
    if (dtype == 0) { SOC_BY_STATE_SIZE(Ns, SOC_SSD_F32) } else { SOC_BY_STATE_SIZE(Ns, SOC_SSD_BF16) }
    return soc_last_error();
}

// ---- causal convolution per channel, then silu -------------------------------------------------------
// y[n, c] = silu(bias[c] + sum_j w[c, j] in(n - (taps - 1) + j)); inputs before the step's first token
// come from the row's state [taps - 1, C], which then becomes the step's last taps - 1 inputs.
// Grid (channel blocks, chunks of CONV_CHUNK tokens, sequences); only a sequence's first chunk
// touches the state (taps - 1 <= CONV_CHUNK), each thread its own channel, reading before writing.
constexpr int CONV_CHUNK = 32;

template <typename T>
__global__ void __launch_bounds__(256)
causal_conv_silu_kernel(const T* __restrict__ x, int ldx, int col, int C, const float* __restrict__ w,
                        const float* __restrict__ bias, int taps, float* __restrict__ state, size_t stride, int offset,
                        const int* __restrict__ seq_qstart, const int* __restrict__ seq_rows, T* __restrict__ out) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int seq = blockIdx.z;
    const int lo = seq_qstart[seq], hi = seq_qstart[seq + 1];
    const int first = lo + blockIdx.y * CONV_CHUNK;
    if (c >= C || first >= hi) return;
    const int last = min(first + CONV_CHUNK, hi);
    float* kept = state + (size_t)seq_rows[seq] * stride + offset;
    const int back = taps - 1;
    for (int n = first; n < last; ++n) {
        float y = bias[c];
        for (int j = 0; j < taps; ++j) {
            const int idx = n - lo - back + j;          // among the step's tokens of this sequence
            const float in = idx >= 0 ? to_float(x[(size_t)(lo + idx) * ldx + col + c])
                                      : kept[(size_t)(back + idx) * C + c];
            y = fmaf(w[(size_t)c * taps + j], in, y);
        }
        out[(size_t)n * C + c] = from_float<T>(y * soc_sigmoid(y));
    }
    if (first == lo) {
        const int len = hi - lo;
        for (int j = 0; j < back; ++j) {                // ascending: entry j + len is read before it is written
            const int idx = len - back + j;
            kept[(size_t)j * C + c] = idx >= 0 ? to_float(x[(size_t)(lo + idx) * ldx + col + c])
                                               : kept[(size_t)(j + len) * C + c];
        }
    }
}

SOC_EXPORT int soc_causal_conv_silu(const void* x, int ldx, int col, int C, const float* w, const float* bias, int taps,
                                    float* state, long long stride, int offset, const int* seq_qstart,
                                    const int* seq_rows, void* out, int n_seqs, int max_q_len, int dtype,
                                    hipStream_t stream) {
    if (n_seqs <= 0 || C <= 0) return 0;
    if (taps < 1 || taps - 1 > CONV_CHUNK) return (int)hipErrorInvalidValue;
    const dim3 grid((C + 255) / 256, (max_q_len + CONV_CHUNK - 1) / CONV_CHUNK, n_seqs);
    if (dtype == 0)
        hipLaunchKernelGGL(causal_conv_silu_kernel<float>, grid, dim3(256), 0, stream, (const float*)x, ldx, col, C, w, bias,
                           taps, state, (size_t)stride, offset, seq_qstart, seq_rows, (float*)out);
    else
        hipLaunchKernelGGL(causal_conv_silu_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)x, ldx, col, C, w, bias,
                           taps, state, (size_t)stride, offset, seq_qstart, seq_rows, (bf16*)out);
    return soc_last_error();
}

// ---- RMS norm in equal parts with a gate silu(z), in front of the norm or behind it ------------------------
// y float32 [N, inner]; z the first `inner` columns of rows of ldz elements. Gate first: norm(y silu(z)) gain;
// gate last: norm(y) gain silu(z). sigmoid_gate: the gate is sigmoid(z) in place of silu(z). An item (part, token) is one wave's (four items to a workgroup), or, for
// parts of 512 elements and more, a whole workgroup's.
template <typename T, bool GATE_FIRST, int WAVES>
__global__ void __launch_bounds__(256)
gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ z, int ldz, const float* __restrict__ gain,
                        int inner, int part, int n_items, float eps, int sigmoid_gate, T* __restrict__ out) {
    __shared__ float scratch[16];
    constexpr int THREADS = WAVES * SOC_WAVE;
    const int item = WAVES == 1 ? blockIdx.x * (256 / SOC_WAVE) + threadIdx.x / SOC_WAVE : blockIdx.x;
    const int lane = threadIdx.x % THREADS;
    if (item >= n_items) return;
    const int parts = inner / part;
    const int n = item / parts, c0 = (item % parts) * part;
    float ss = 0.f;
    for (int c = c0 + lane; c < c0 + part; c += THREADS) {
        float v = y[(size_t)n * inner + c];
        if (GATE_FIRST) { const float zz = to_float(z[(size_t)n * ldz + c]); v *= sigmoid_gate ? soc_sigmoid(zz) : zz * soc_sigmoid(zz); }
        ss += v * v;
    }
    ss = WAVES == 1 ? wave_sum(ss) : block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)part + eps);
    for (int c = c0 + lane; c < c0 + part; c += THREADS) {
        const float zz = to_float(z[(size_t)n * ldz + c]);
        const float v = y[(size_t)n * inner + c] * (sigmoid_gate ? soc_sigmoid(zz) : zz * soc_sigmoid(zz));
        out[(size_t)n * inner + c] = from_float<T>(v * inv * gain[c]);
    }
}

SOC_EXPORT int soc_gated_group_norm(const float* y, const void* z, int ldz, const float* gain, int N, int inner, int parts,
                                    float eps, int gate_first, int sigmoid_gate, void* out, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (parts < 1 || inner % parts || (long long)N * parts > 0x7fffffffLL) return (int)hipErrorInvalidValue;
    const int items = N * parts;
    const bool wide = inner / parts >= 512;
    const dim3 grid(wide ? items : (items + 3) / 4);
#define SOC_GGN(T, FIRST, WAVES)                                                                                              \
    hipLaunchKernelGGL((gated_group_norm_kernel<T, FIRST, WAVES>), grid, dim3(256), 0, stream, y, (const T*)z, ldz, gain, inner, \
                       inner / parts, items, eps, sigmoid_gate, (T*)out)
#define SOC_GGN_T(T)                                                                                   \
    if (gate_first) { if (wide) SOC_GGN(T, true, 4); else SOC_GGN(T, true, 1); }                       \
    else { if (wide) SOC_GGN(T, false, 4); else SOC_GGN(T, false, 1); }
    if (dtype == 0) { SOC_GGN_T(float) } else { SOC_GGN_T(bf16) }
    return soc_last_error();
}

// ---- RMS norm of the first dim elements of rows of ld elements, into rows of dim -------------------------------
// (a query latent that is some of the columns of a wider product). One wave per row.
template <typename T>
__global__ void __launch_bounds__(256)
rmsnorm_cols_kernel(const T* __restrict__ x, int ld, const float* __restrict__ w, T* __restrict__ out, int N, int dim,
                    float eps) {
    const int n = blockIdx.x * (256 / SOC_WAVE) + threadIdx.x / SOC_WAVE, lane = threadIdx.x % SOC_WAVE;
    if (n >= N) return;
    const T* row = x + (size_t)n * ld;
    float ss = 0.f;
    for (int c = lane; c < dim; c += SOC_WAVE) { const float v = to_float(row[c]); ss += v * v; }
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)dim + eps);
    for (int c = lane; c < dim; c += SOC_WAVE) out[(size_t)n * dim + c] = from_float<T>(to_float(row[c]) * inv * w[c]);
}

SOC_EXPORT int soc_rmsnorm_cols(const void* x, int ld, const float* w, void* out, int N, int dim, float eps, int dtype,
                                hipStream_t stream) {
    if (N <= 0) return 0;
    if (dim < 1 || ld < dim) return (int)hipErrorInvalidValue;
    const dim3 grid((N + 3) / 4);
    if (dtype == 0)
        hipLaunchKernelGGL(rmsnorm_cols_kernel<float>, grid, dim3(256), 0, stream, (const float*)x, ld, w, (float*)out, N, dim, eps);
    else
        hipLaunchKernelGGL(rmsnorm_cols_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)x, ld, w, (bf16*)out, N, dim, eps);
    return soc_last_error();
}

// ---- a token's latent into its page ---------------------------------------------------------------------------
// kvd: the first R + Dr elements of rows of ld elements: the first R RMS-normed with gain, the rest turned pair by pair (pairs 2i, 2i + 1 of the
// first 2 * half by position * inv_freq[i]); both go to the token's place in the pool
// [pages, 1, block, width], the padding up to width as zeros. One wave per token.
template <typename T>
__global__ void __launch_bounds__(64)
latent_write_kernel(const T* __restrict__ kvd, int ld, int R, int Dr, const float* __restrict__ gain, float eps,
                    const float* __restrict__ inv_freq, int half, const int* __restrict__ positions,
                    const int* __restrict__ token_rows, const int* __restrict__ table, int table_width,
                    T* __restrict__ pool, int block, int width) {
    const int n = blockIdx.x, lane = threadIdx.x;
    const T* row = kvd + (size_t)n * ld;
    const int pos = positions[n];
    const int page = table[(size_t)token_rows[n] * table_width + pos / block];
    T* dst = pool + ((size_t)page * block + pos % block) * width;
    float ss = 0.f;
    for (int c = lane; c < R; c += 64) { const float v = to_float(row[c]); ss += v * v; }
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)R + eps);
    for (int c = lane; c < R; c += 64) dst[c] = from_float<T>(to_float(row[c]) * inv * gain[c]);
    for (int i = lane; i < Dr / 2; i += 64) {
        const float a = to_float(row[R + 2 * i]), b = to_float(row[R + 2 * i + 1]);
        if (i < half) {
            float sn, cs;
            sincosf((float)pos * inv_freq[i], &sn, &cs);
            dst[R + 2 * i] = from_float<T>(a * cs - b * sn);
            dst[R + 2 * i + 1] = from_float<T>(b * cs + a * sn);
        } else {
            dst[R + 2 * i] = from_float<T>(a);
            dst[R + 2 * i + 1] = from_float<T>(b);
        }
    }
    if (lane == 0 && (Dr & 1)) dst[R + Dr - 1] = row[R + Dr - 1];
    for (int c = R + Dr + lane; c < width; c += 64) dst[c] = from_float<T>(0.f);
}

SOC_EXPORT int soc_latent_write(const void* kvd, int ld, int N, int R, int Dr, const float* gain, float eps, const float* inv_freq,
                                int half, const int* positions, const int* token_rows, const int* table, int table_width,
                                void* pool, int block, int width, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (2 * half > Dr || R + Dr > width || ld < R + Dr) return (int)hipErrorInvalidValue;
    if (dtype == 0)
        hipLaunchKernelGGL(latent_write_kernel<float>, dim3(N), dim3(64), 0, stream, (const float*)kvd, ld, R, Dr, gain, eps, inv_freq,
                           half, positions, token_rows, table, table_width, (float*)pool, block, width);
    else
        hipLaunchKernelGGL(latent_write_kernel<bf16>, dim3(N), dim3(64), 0, stream, (const bf16*)kvd, ld, R, Dr, gain, eps, inv_freq,
                           half, positions, token_rows, table, table_width, (bf16*)pool, block, width);
    return soc_last_error();
}

// ---- the rotated part of every head's query, beside the folded plain part ---------------------------------------
// q [N, H, D + Dr] -> out [N, H, width]: out[.., R : R + Dr] = turned q[.., D :], zeros behind it.
// (out[.., : R] is written by the product per head.) One thread per (token, head, pair or padding element).
template <typename T>
__global__ void latent_query_turn_kernel(const T* __restrict__ q, int H, int D, int Dr, int R, int width,
                                         const float* __restrict__ inv_freq, int half, const int* __restrict__ positions,
                                         T* __restrict__ out, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int per = width - R;                      // elements behind the folded part
    const int e = (int)(i % per);
    const size_t nh = i / per;
    const int n = (int)(nh / H);
    const T* src = q + nh * (D + Dr) + D;
    T* dst = out + nh * width + R;
    if (e >= Dr) { dst[e] = from_float<T>(0.f); return; }
    const int pair = e / 2;
    if (pair >= half || (e | 1) >= Dr) { dst[e] = src[e]; return; }
    float sn, cs;
    sincosf((float)positions[n] * inv_freq[pair], &sn, &cs);
    const float a = to_float(src[2 * pair]), b = to_float(src[2 * pair + 1]);
    dst[e] = from_float<T>((e & 1) ? b * cs + a * sn : a * cs - b * sn);
}

SOC_EXPORT int soc_latent_query_turn(const void* q, int N, int H, int D, int Dr, int R, int width, const float* inv_freq,
                                     int half, const int* positions, void* out, int dtype, hipStream_t stream) {
    const size_t total = (size_t)N * H * (width - R);
    if (total == 0) return 0;
    if (2 * half > Dr || R + Dr > width) return (int)hipErrorInvalidValue;
    const dim3 grid((unsigned)((total + 255) / 256));
    if (dtype == 0)
        hipLaunchKernelGGL(latent_query_turn_kernel<float>, grid, dim3(256), 0, stream, (const float*)q, H, D, Dr, R, width,
                           inv_freq, half, positions, (float*)out, total);
    else
        hipLaunchKernelGGL(latent_query_turn_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)q, H, D, Dr, R, width,
                           inv_freq, half, positions, (bf16*)out, total);
    return soc_last_error();
}

// ---- one small product per head ------------------------------------------------------------------------------------
// out[n, h, o] = sum_k x[n, h, k] w[h, o, k], k < K, o < n_out; x rows of ldx elements per head (its first K are
// read), out rows of ldo elements per head (its first n_out are written). Tiles of 16 tokens x 64 outputs,
// 32 k at a time through LDS; float32 sums, k in order.
template <typename T>
__global__ void __launch_bounds__(256)
head_linear_kernel(const T* __restrict__ x, int ldx, const T* __restrict__ w, T* __restrict__ out, int ldo,
                   int N, int H, int n_out, int K) {
    __shared__ float xs[16][33], ws[64][33];
    const int head = blockIdx.z, n0 = blockIdx.y * 16, o0 = blockIdx.x * 64;
    const int to = threadIdx.x % 64, tn = threadIdx.x / 64;          // output column; token group of 4
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += 32) {
        for (int e = threadIdx.x; e < 16 * 32; e += 256) {
            const int rn = e / 32, rk = e % 32;
            xs[rn][rk] = (n0 + rn < N && k0 + rk < K) ? to_float(x[((size_t)(n0 + rn) * H + head) * ldx + k0 + rk]) : 0.f;
        }
        for (int e = threadIdx.x; e < 64 * 32; e += 256) {
            const int ro = e / 32, rk = e % 32;
            ws[ro][rk] = (o0 + ro < n_out && k0 + rk < K) ? to_float(w[((size_t)head * n_out + o0 + ro) * K + k0 + rk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 32; ++kk) {
            const float wv = ws[to][kk];
#pragma unroll
            for (int t = 0; t < 4; ++t) acc[t] = fmaf(xs[tn * 4 + t][kk], wv, acc[t]);
        }
        __syncthreads();
    }
    if (o0 + to < n_out)
        for (int t = 0; t < 4; ++t)
            if (n0 + tn * 4 + t < N)
                out[((size_t)(n0 + tn * 4 + t) * H + head) * ldo + o0 + to] = from_float<T>(acc[t]);
}

// The same product for steps of at most 16 tokens, where the tiles above would wait for memory once per 32 k:
// a wave per (head, output), its lanes over k, all loads issued at once, one sum over the wave per token.
template <typename T>
__global__ void __launch_bounds__(256)
head_linear_rows_kernel(const T* __restrict__ x, int ldx, const T* __restrict__ w, T* __restrict__ out, int ldo,
                        int N, int H, int n_out, int K) {
    const int head = blockIdx.y, o = blockIdx.x * 4 + threadIdx.x / SOC_WAVE, lane = threadIdx.x % SOC_WAVE;
    if (o >= n_out) return;
    float acc[16];
#pragma unroll
    for (int n = 0; n < 16; ++n) acc[n] = 0.f;
    const T* wrow = w + ((size_t)head * n_out + o) * K;
    for (int k = lane; k < K; k += SOC_WAVE) {
        const float wv = to_float(wrow[k]);
#pragma unroll
        for (int n = 0; n < 16; ++n)
            if (n < N) acc[n] = fmaf(to_float(x[((size_t)n * H + head) * ldx + k]), wv, acc[n]);
    }
#pragma unroll
    for (int n = 0; n < 16; ++n) {
        if (n < N) {
            const float sum = wave_sum(acc[n]);
            if (lane == 0) out[((size_t)n * H + head) * ldo + o] = from_float<T>(sum);
        }
    }
}

SOC_EXPORT int soc_head_linear(const void* x, int ldx, const void* w, void* out, int ldo, int N, int H, int n_out, int K,
                               int dtype, hipStream_t stream) {
    if (N <= 0 || H <= 0 || n_out <= 0) return 0;
    if (K < 1 || K > ldx || n_out > ldo || H > 65535 || (N + 15) / 16 > 65535) return (int)hipErrorInvalidValue;
    if (N <= 16) {
        const dim3 rows_grid((n_out + 3) / 4, H);
        if (dtype == 0)
            hipLaunchKernelGGL(head_linear_rows_kernel<float>, rows_grid, dim3(256), 0, stream, (const float*)x, ldx,
                               (const float*)w, (float*)out, ldo, N, H, n_out, K);
        else
            hipLaunchKernelGGL(head_linear_rows_kernel<bf16>, rows_grid, dim3(256), 0, stream, (const bf16*)x, ldx,
                               (const bf16*)w, (bf16*)out, ldo, N, H, n_out, K);
        return soc_last_error();
    }
    const dim3 grid((n_out + 63) / 64, (N + 15) / 16, H);
    if (dtype == 0)
        hipLaunchKernelGGL(head_linear_kernel<float>, grid, dim3(256), 0, stream, (const float*)x, ldx, (const float*)w,
                           (float*)out, ldo, N, H, n_out, K);
    else
        hipLaunchKernelGGL(head_linear_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)x, ldx, (const bf16*)w,
                           (bf16*)out, ldo, N, H, n_out, K);
    return soc_last_error();
}
