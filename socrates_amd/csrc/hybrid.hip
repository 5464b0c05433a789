// Kernels of layers that mix kinds: what prepares attention whose keys and values differ in size
// (per-head norm, partial rotation, a blend of the values with an earlier layer's, page writes
// padded to the pools' head size), a gate per head behind it, retention (linear attention with a
// fixed decay per head and a matrix state), routed experts (choice among groups, sorting tokens
// by expert, products per expert, the weighted sum), the squared-relu activation, a per-token
// side input, and the sum into the residual stream with a cast.
//
// Statistics, angles, routers, the recurrence and its state and the residual sum are float32
// whatever the compute dtype; a value is rounded once, where it is stored in the compute dtype.
#include "common.h"
#include "recurrent.h"

__device__ __forceinline__ float hyb_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }

// ---- per-head norm, rotation, value blend and page write ------------------------------------------
// x: rows of ld elements that hold, from col_q / col_k / col_v on, Hq heads of D, Hkv heads of D and
// Hkv heads of Dv. One wave per (token, head): q heads are RMS-normed over D (gain, eps), turned over
// their first 2 * half elements (element i pairs with i + half; angle position * inv_freq[i]) and
// written to q_out [N, Hq, P], zeros from D on; k heads the same, into the token's place of the pool
// [pages, Hkv, BS, P]; v heads become (1 - lam) v + lam first (first: rows of ldf elements, the values
// of an earlier layer for the same token; lam one stored number) if first is given, and go to their
// pool, zeros from Dv on. D, Dv <= P <= 256.
template <typename T>
__global__ void __launch_bounds__(256)
attn_prepare_kernel(const T* __restrict__ x, int ld, int col_q, int col_k, int col_v, const T* __restrict__ first, int ldf,
                    const float* __restrict__ lam, T* __restrict__ q_out, T* __restrict__ k_pool, T* __restrict__ v_pool,
                    const int* __restrict__ table, int table_width, const int* __restrict__ token_rows,
                    const int* __restrict__ positions, const float* __restrict__ q_gain, const float* __restrict__ k_gain,
                    const float* __restrict__ inv_freq, int N, int Hq, int Hkv, int D, int Dv, int P, int half, int BS,
                    float eps) {
    __shared__ float normed[4][256];
    const int wave = threadIdx.x / SOC_WAVE, lane = threadIdx.x % SOC_WAVE;
    const int items = Hq + 2 * Hkv;
    const long long item = (long long)blockIdx.x * 4 + wave;
    if (item >= (long long)N * items) return;
    const int n = (int)(item / items), h = (int)(item % items);
    const int pos = positions[n];
    const T* row = x + (size_t)n * ld;
    T* dst = nullptr;
    if (h >= Hq) {
        const int page = table[(size_t)token_rows[n] * table_width + pos / BS];
        const int kvh = h < Hq + Hkv ? h - Hq : h - Hq - Hkv;
        dst = (h < Hq + Hkv ? k_pool : v_pool) + (((size_t)page * Hkv + kvh) * BS + pos % BS) * P;
    } else {
        dst = q_out + ((size_t)n * Hq + h) * P;
    }
    if (h >= Hq + Hkv) {                                   // a value head
        const int kvh = h - Hq - Hkv;
        const float l = first ? lam[0] : 0.f;
        for (int i = lane; i < P; i += SOC_WAVE) {
            float v = 0.f;
            if (i < Dv) {
                v = to_float(row[col_v + kvh * Dv + i]);
                if (first) v = (1.f - l) * v + l * to_float(first[(size_t)n * ldf + kvh * Dv + i]);
            }
            dst[i] = from_float<T>(v);
        }
        return;
    }
    const bool is_q = h < Hq;
    const T* src = row + (is_q ? col_q + h * D : col_k + (h - Hq) * D);
    const float* gain = is_q ? q_gain : k_gain;
    float xv[4], ss = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int i = lane + j * SOC_WAVE;
        xv[j] = i < D ? to_float(src[i]) : 0.f;
        ss = fmaf(xv[j], xv[j], ss);
    }
    if (gain) {
        const float r = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = lane + j * SOC_WAVE;
            if (i < D) xv[j] = xv[j] * r * gain[i];
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int i = lane + j * SOC_WAVE;
        if (i < D) normed[wave][i] = xv[j];
    }
    __builtin_amdgcn_wave_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int i = lane + j * SOC_WAVE;
        if (i >= P) break;
        float y = 0.f;
        if (i < D) {
            y = xv[j];
            if (i < 2 * half) {
                const int f = i < half ? i : i - half;
                float sn, cs;
                sincosf((float)pos * inv_freq[f], &sn, &cs);
                y = i < half ? xv[j] * cs - normed[wave][i + half] * sn : xv[j] * cs + normed[wave][i - half] * sn;
            }
        }
        dst[i] = from_float<T>(y);
    }
}

SOC_EXPORT int soc_attn_prepare(const void* x, int ld, int col_q, int col_k, int col_v, const void* first, int ldf,
                                const float* lam, void* q_out, void* k_pool, void* v_pool, const int* table, int table_width,
                                const int* token_rows, const int* positions, const float* q_gain, const float* k_gain,
                                const float* inv_freq, int N, int Hq, int Hkv, int D, int Dv, int P, int half, int BS,
                                float eps, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (D < 1 || Dv < 1 || D > P || Dv > P || P > 256 || 2 * half > D || BS < 1) return (int)hipErrorInvalidValue;
    const long long items = (long long)N * (Hq + 2 * Hkv);
    const dim3 grid((unsigned)((items + 3) / 4));
#define SOC_PREP(T)                                                                                                           \
    hipLaunchKernelGGL(attn_prepare_kernel<T>, grid, dim3(256), 0, stream, (const T*)x, ld, col_q, col_k, col_v,              \
                       (const T*)first, ldf, lam, (T*)q_out, (T*)k_pool, (T*)v_pool, table, table_width, token_rows,          \
                       positions, q_gain, k_gain, inv_freq, N, Hq, Hkv, D, Dv, P, half, BS, eps)
    if (dtype == 0) SOC_PREP(float); else SOC_PREP(bf16);
#undef SOC_PREP
    return soc_last_error();
}

// ---- a gate per head ---------------------------------------------------------------------------------
// out[n, h, j] = o[n, h, j] * sigmoid(g[n, h]), j < Dv; o rows of P elements per head, g rows of ldg
// (g null: the first Dv elements of each head as they are).
template <typename T>
__global__ void head_gate_kernel(const T* __restrict__ o, const T* __restrict__ g, int ldg, T* __restrict__ out, size_t total,
                                 int H, int P, int Dv) {
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const int j = (int)(e % Dv);
        const size_t nh = e / Dv;
        const int h = (int)(nh % H);
        const size_t n = nh / H;
        out[e] = from_float<T>(to_float(o[nh * P + j]) * (g ? hyb_sigmoid(to_float(g[n * ldg + h])) : 1.f));
    }
}

SOC_EXPORT int soc_head_gate(const void* o, const void* g, int ldg, void* out, int N, int H, int P, int Dv, int dtype,
                             hipStream_t stream) {
    const size_t total = (size_t)N * H * Dv;
    if (!total) return 0;
    const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    if (dtype == 0)
        hipLaunchKernelGGL(head_gate_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)o, (const float*)g, ldg,
                           (float*)out, total, H, P, Dv);
    else
        hipLaunchKernelGGL(head_gate_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)o, (const bf16*)g, ldg,
                           (bf16*)out, total, H, P, Dv);
    return soc_last_error();
}

// ---- retention: S <- decay S + k v^T, o = S^T q, a fixed decay per head -------------------------------------
// x: rows of ld elements with H heads of D (q, from col_q; k, from col_k) and H heads of Dv (v, from col_v).
// q and k are turned over their first 2 * half elements by the token's position and k is scaled, in float32,
// while a batch of tokens is staged, or ahead of the walk by a kernel of its own (turned: [N, 2, H * D] float32;
// every workgroup of a head's columns would turn the head's q and k again, which costs a long portion more than
// the walk itself). The state [H, D, Dv] of the sequence's row is float32; a workgroup owns CW columns of one
// head, thread (part, column) a slice of the keys. o goes out in float32 [N, H * Dv].
// q and k of every token turned by its position over their first 2 * half elements and k scaled, float32:
// turned [N, 2, H * D]. One thread per (token, head, pair) and per element behind the turned part.
template <typename T>
__global__ void retention_turn_kernel(const T* __restrict__ x, int ld, int col_q, int col_k, const int* __restrict__ positions,
                                      const float* __restrict__ inv_freq, int half, float k_scale, int H, int D, size_t total,
                                      float* __restrict__ turned) {
    const int per = half + (D - 2 * half);                 // work items of one head: pairs, then single elements
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const int w = (int)(e % per);
        const size_t nh = e / per;
        const int h = (int)(nh % H);
        const size_t n = nh / H;
        const T* row = x + n * ld + h * D;
        float* q = turned + n * 2 * H * D + (size_t)h * D;
        float* k = q + (size_t)H * D;
        if (w < half) {
            const float a = to_float(row[col_q + w]), b = to_float(row[col_q + w + half]);
            const float a2 = to_float(row[col_k + w]), b2 = to_float(row[col_k + w + half]);
            float sn, cs;
            sincosf((float)positions[n] * inv_freq[w], &sn, &cs);
            q[w] = a * cs - b * sn; q[w + half] = b * cs + a * sn;
            k[w] = (a2 * cs - b2 * sn) * k_scale; k[w + half] = (b2 * cs + a2 * sn) * k_scale;
        } else {
            const int d = 2 * half + (w - half);
            q[d] = to_float(row[col_q + d]);
            k[d] = to_float(row[col_k + d]) * k_scale;
        }
    }
}

template <typename T, int DK, int CW>
__global__ void __launch_bounds__(256)
retention_kernel(const T* __restrict__ x, int ld, int col_q, int col_k, int col_v, const int* __restrict__ positions,
                 const float* __restrict__ inv_freq, int half, float k_scale, const float* __restrict__ decays, int H, int D,
                 int Dv, float* __restrict__ state, size_t stride, int offset, const int* __restrict__ seq_qstart,
                 const int* __restrict__ seq_rows, const float* __restrict__ turned, float* __restrict__ out) {
    constexpr int REC_TB = rec_batch(DK), PARTS = 256 / CW, KPT = DK / PARTS, STAGE = (REC_TB * DK + 255) / 256;
    __shared__ float sq[2][REC_TB][DK], sk[2][REC_TB][DK];
    __shared__ float red[REC_TB][PARTS][CW];
    const int blocks = (Dv + CW - 1) / CW;
    const int head = blockIdx.x / blocks, seq = blockIdx.y, tid = threadIdx.x;
    const int lo = seq_qstart[seq], hi = seq_qstart[seq + 1];
    if (lo >= hi) return;
    const int col0 = (blockIdx.x % blocks) * CW;
    const int col = col0 + tid % CW, part = tid / CW, i0 = part * KPT;
    const bool live = col < Dv;
    float* S = state + (size_t)seq_rows[seq] * stride + offset + (size_t)head * D * Dv;
    const float decay = decays[head];
    float s[KPT];
#pragma unroll
    for (int ii = 0; ii < KPT; ++ii) s[ii] = (live && i0 + ii < D) ? S[(size_t)(i0 + ii) * Dv + col] : 0.f;

    float fq[STAGE], fk[STAGE], fv[REC_TB];
    auto fetch = [&](int n0) {
#pragma unroll
        for (int q = 0; q < STAGE; ++q) {
            const int e = tid + q * 256, t = e / DK, i = e % DK;
            const bool in = t < REC_TB && n0 + t < hi && i < D;
            float a = 0.f, b = 0.f;
            if (in && turned) {                        // q and k were turned and scaled ahead, [N, 2, H * D] float32
                const float* row = turned + (size_t)(n0 + t) * 2 * H * D + head * D + i;
                a = row[0];
                b = row[(size_t)H * D];
            } else if (in) {
                const T* row = x + (size_t)(n0 + t) * ld + head * D;
                a = to_float(row[col_q + i]);
                b = to_float(row[col_k + i]);
                if (i < 2 * half) {
                    const int f = i < half ? i : i - half, other = i < half ? i + half : i - half;
                    const float a2 = to_float(row[col_q + other]), b2 = to_float(row[col_k + other]);
                    float sn, cs;
                    sincosf((float)positions[n0 + t] * inv_freq[f], &sn, &cs);
                    if (i < half) { a = a * cs - a2 * sn; b = b * cs - b2 * sn; }
                    else          { a = a * cs + a2 * sn; b = b * cs + b2 * sn; }
                }
                b *= k_scale;
            }
            fq[q] = a;
            fk[q] = b;
        }
#pragma unroll
        for (int t = 0; t < REC_TB; ++t)
            fv[t] = (live && n0 + t < hi) ? to_float(x[(size_t)(n0 + t) * ld + col_v + head * Dv + col]) : 0.f;
    };
    auto land = [&](int buf) {
#pragma unroll
        for (int q = 0; q < STAGE; ++q) {
            const int e = tid + q * 256, t = e / DK, i = e % DK;
            if (t < REC_TB) { sq[buf][t][i] = fq[q]; sk[buf][t][i] = fk[q]; }
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
                    s[ii] = fmaf(decay, s[ii], sk[buf][t][i0 + ii] * vj[t]);
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
static void launch_retention(const void* x, int ld, int col_q, int col_k, int col_v, const int* positions, const float* inv_freq,
                             int half, float k_scale, const float* decays, int H, int D, int Dv, float* state, long long stride,
                             int offset, const int* seq_qstart, const int* seq_rows, const float* turned, float* out, int n_seqs,
                             int cw, hipStream_t stream) {
#define SOC_RET_LAUNCH(CW)                                                                                                     \
    hipLaunchKernelGGL((retention_kernel<T, DK, CW>), dim3(H * ((Dv + CW - 1) / CW), n_seqs), dim3(256), 0, stream,            \
                       (const T*)x, ld, col_q, col_k, col_v, positions, inv_freq, half, k_scale, decays, H, D, Dv, state,      \
                       (size_t)stride, offset, seq_qstart, seq_rows, turned, out)
    if (cw == 16) SOC_RET_LAUNCH(16); else SOC_RET_LAUNCH(64);
#undef SOC_RET_LAUNCH
}

SOC_EXPORT int soc_retention(const void* x, int ld, int col_q, int col_k, int col_v, const int* positions, const float* inv_freq,
                             int half, float k_scale, const float* decays, int H, int D, int Dv, float* state, long long stride,
                             int offset, const int* seq_qstart, const int* seq_rows, float* turned, int n_tokens, float* out,
                             int n_seqs, int max_q_len, int dtype, hipStream_t stream) {
    if (n_seqs <= 0 || H <= 0) return 0;
    if (D < 1 || D > 256 || Dv < 1 || n_seqs > 65535 || 2 * half > D) return (int)hipErrorInvalidValue;
    if (turned) {                                          // scratch [n_tokens, 2, H * D]: turn q and k ahead of the walk
        const size_t total = (size_t)n_tokens * H * (D - half);
        const int blocks = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
        if (dtype == 0)
            hipLaunchKernelGGL(retention_turn_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)x, ld, col_q, col_k,
                               positions, inv_freq, half, k_scale, H, D, total, turned);
        else
            hipLaunchKernelGGL(retention_turn_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)x, ld, col_q, col_k,
                               positions, inv_freq, half, k_scale, H, D, total, turned);
    }
    const int cw = columns_per_workgroup(H, Dv, n_seqs, max_q_len);
#define SOC_RET_F32(DK) launch_retention<float, DK>(x, ld, col_q, col_k, col_v, positions, inv_freq, half, k_scale, decays, H, D, Dv, state, stride, offset, seq_qstart, seq_rows, turned, out, n_seqs, cw, stream)
#define SOC_RET_BF16(DK) launch_retention<bf16, DK>(x, ld, col_q, col_k, col_v, positions, inv_freq, half, k_scale, decays, H, D, Dv, state, stride, offset, seq_qstart, seq_rows, turned, out, n_seqs, cw, stream)
    if (dtype == 0) { SOC_BY_STATE_SIZE(D, SOC_RET_F32) } else { SOC_BY_STATE_SIZE(D, SOC_RET_BF16) }
    return soc_last_error();
}

// ---- relu(x)^2 ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void relu_squared_kernel(const T* __restrict__ x, T* __restrict__ out, size_t total) {
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const float v = fmaxf(to_float(x[e]), 0.f);
        out[e] = from_float<T>(v * v);
    }
}

SOC_EXPORT int soc_relu_squared(const void* x, void* out, long long total, int dtype, hipStream_t stream) {
    if (total <= 0) return 0;
    const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
    if (dtype == 0)
        hipLaunchKernelGGL(relu_squared_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)x, (float*)out, (size_t)total);
    else
        hipLaunchKernelGGL(relu_squared_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)x, (bf16*)out, (size_t)total);
    return soc_last_error();
}

// ---- the choice of experts ----------------------------------------------------------------------------------
// One wave per token. s = softmax(z) over E experts (E <= 256), or sigmoid(z) each; z rows are ldz apart; choice
// scores c = s + correction (if given). Experts lie in n_groups equal groups of neighbours; a group's score is the
// sum of its group_top largest c (1: its largest); the weights are multiplied by scale; only experts of the
// keep_groups best groups can be chosen (n_groups <= 1: all). The top experts by c (the lower index among
// equals) are chosen; their weights are their s over the sum of the chosen s (+ renorm_eps).
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const float v2 = __shfl_xor(v, m, SOC_WAVE);
        const int i2 = __shfl_xor(i, m, SOC_WAVE);
        if (v2 > v || (v2 == v && i2 < i)) { v = v2; i = i2; }
    }
}

__global__ void __launch_bounds__(256)
moe_route_kernel(const float* __restrict__ z, int ldz, const float* __restrict__ correction, int N, int E, int top, int n_groups,
                 int keep_groups, float renorm_eps, int sigmoid, int group_top, float scale, int* __restrict__ idx,
                 float* __restrict__ weight) {
    __shared__ float sc[4][256];
    __shared__ float ss[4][256];
    const int wave = threadIdx.x / SOC_WAVE, lane = threadIdx.x % SOC_WAVE;
    const int n = blockIdx.x * 4 + wave;
    if (n >= N) return;
    float zv[4], m = -INFINITY;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = lane + j * SOC_WAVE;
        zv[j] = e < E ? z[(size_t)n * ldz + e] : -INFINITY;
        m = fmaxf(m, zv[j]);
    }
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (sigmoid) zv[j] = lane + j * SOC_WAVE < E ? hyb_sigmoid(zv[j]) : 0.f;
        else zv[j] = lane + j * SOC_WAVE < E ? expf(zv[j] - m) : 0.f;
        sum += zv[j];
    }
    sum = sigmoid ? 1.f : wave_sum(sum);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = lane + j * SOC_WAVE;
        if (e < E) {
            const float s = zv[j] / sum;
            ss[wave][e] = s;
            sc[wave][e] = correction ? s + correction[e] : s;
        }
    }
    __builtin_amdgcn_wave_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (n_groups > 1 && keep_groups < n_groups) {
        const int per = E / n_groups;
        float gs[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int g = lane + j * SOC_WAVE;
            gs[j] = -INFINITY;
            if (g < n_groups && group_top <= 1)
                for (int e = g * per; e < (g + 1) * per; ++e) gs[j] = fmaxf(gs[j], sc[wave][e]);
            if (g < n_groups && group_top > 1) {
                // the group_top largest, one after the other: each the largest that comes behind the last one
                // taken in the order (score falling, index rising)
                float pv = INFINITY, acc = 0.f;
                int pi = -1;
                for (int r = 0; r < group_top && r < per; ++r) {
                    float bv = -INFINITY;
                    int bi = -1;
                    for (int e = g * per; e < (g + 1) * per; ++e) {
                        const float v = sc[wave][e];
                        const bool behind = v < pv || (v == pv && e > pi);
                        if (behind && (bi < 0 || v > bv)) { bv = v; bi = e; }
                    }
                    if (bi < 0) break;
                    acc += bv; pv = bv; pi = bi;
                }
                gs[j] = acc;
            }
        }
        bool kept[4] = {false, false, false, false};
        for (int r = 0; r < keep_groups; ++r) {
            float bv = -INFINITY;
            int bi = 0x7fffffff;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int g = lane + j * SOC_WAVE;
                if (g < n_groups && !kept[j] && (gs[j] > bv || (gs[j] == bv && g < bi))) { bv = gs[j]; bi = g; }
            }
            wave_argmax(bv, bi);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (lane + j * SOC_WAVE == bi) kept[j] = true;
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int g = lane + j * SOC_WAVE;
            if (g < n_groups && !kept[j])
                for (int e = g * per; e < (g + 1) * per; ++e) sc[wave][e] = -INFINITY;
        }
        __builtin_amdgcn_wave_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    float cv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) cv[j] = lane + j * SOC_WAVE < E ? sc[wave][lane + j * SOC_WAVE] : -INFINITY;
    bool taken[4] = {false, false, false, false};
    float total = 0.f;
    for (int r = 0; r < top; ++r) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = lane + j * SOC_WAVE;
            if (e < E && !taken[j] && (cv[j] > bv || (cv[j] == bv && e < bi))) { bv = cv[j]; bi = e; }
        }
        wave_argmax(bv, bi);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (lane + j * SOC_WAVE == bi) taken[j] = true;
        total += ss[wave][bi];
        if (lane == 0) { idx[(size_t)n * top + r] = bi; sc[wave][r] = ss[wave][bi]; }     // (sc is free: cv holds it)
    }
    if (lane == 0)
        for (int r = 0; r < top; ++r) weight[(size_t)n * top + r] = sc[wave][r] / (total + renorm_eps) * scale;
}

SOC_EXPORT int soc_moe_route(const float* z, int ldz, const float* correction, int N, int E, int top, int n_groups, int keep_groups,
                             float renorm_eps, int sigmoid, int group_top, float scale, int* idx, float* weight,
                             hipStream_t stream) {
    if (N <= 0) return 0;
    if (E < 1 || E > 256 || ldz < E || group_top < 1 || top < 1 || top > E || n_groups < 1 || E % n_groups || keep_groups < 1 || keep_groups > n_groups ||
        (long long)keep_groups * (E / n_groups) < top)
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(moe_route_kernel, dim3((N + 3) / 4), dim3(256), 0, stream, z, ldz, correction, N, E, top, n_groups,
                       keep_groups, renorm_eps, sigmoid, group_top, scale, idx, weight);
    return soc_last_error();
}

// ---- tokens sorted by expert ----------------------------------------------------------------------------------
// idx [M] (M = tokens x top): the expert of each (token, choice) pair. One workgroup counts the pairs of each
// expert, lays the experts' runs one after the other (offsets [E + 1]), gives each pair its place (place [M]) and
// each place its pair (pair_at [M]), and lists the tiles of TM places that the products walk: tiles [max_tiles, 2]
// = (expert, first place), expert -1 behind the last tile. max_tiles >= M / TM + E.
__global__ void __launch_bounds__(1024)
moe_sort_kernel(const int* __restrict__ idx, int M, int E, int TM, int max_tiles, int* __restrict__ offsets,
                int* __restrict__ place, int* __restrict__ pair_at, int* __restrict__ tiles) {
    __shared__ int count[256], start[257], cursor[256], tile0[257];
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += 1024) count[e] = 0;
    __syncthreads();
    for (int i = tid; i < M; i += 1024) atomicAdd(&count[idx[i]], 1);
    __syncthreads();
    if (tid == 0) {
        int at = 0, t = 0;
        for (int e = 0; e < E; ++e) {
            start[e] = at; tile0[e] = t;
            at += count[e];
            t += (count[e] + TM - 1) / TM;
        }
        start[E] = at; tile0[E] = t;
    }
    __syncthreads();
    for (int e = tid; e <= E; e += 1024) offsets[e] = start[e];
    for (int e = tid; e < E; e += 1024) cursor[e] = start[e];
    __syncthreads();
    for (int i = tid; i < M; i += 1024) {
        const int at = atomicAdd(&cursor[idx[i]], 1);
        place[i] = at;
        pair_at[at] = i;
    }
    for (int t = tid; t < max_tiles; t += 1024) {
        int e = -1, first = 0;
        if (t < tile0[E]) {
            int lo = 0, hi = E - 1;                      // the last expert whose first tile is <= t and that has tiles
            while (lo < hi) {
                const int mid = (lo + hi + 1) / 2;
                if (tile0[mid] <= t) lo = mid; else hi = mid - 1;
            }
            e = lo;
            first = start[e] + (t - tile0[e]) * TM;
        }
        tiles[2 * t] = e;
        tiles[2 * t + 1] = first;
    }
}

SOC_EXPORT int soc_moe_sort(const int* idx, int M, int E, int TM, int max_tiles, int* offsets, int* place, int* pair_at,
                            int* tiles, hipStream_t stream) {
    if (M <= 0) return 0;
    if (E < 1 || E > 256 || TM < 1 || max_tiles < (M + TM - 1) / TM + (E < M ? E : M)) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, idx, M, E, TM, max_tiles, offsets, place, pair_at, tiles);
    return soc_last_error();
}

// ---- products per expert -----------------------------------------------------------------------------------------
// out[p, o] = sum_k x[src(p), k] w[e, o, k] for the places p of expert e's run, o < n_out. src(p) = pair_at[p] / top
// (rows of x are tokens) if pair_at is given, else p (rows of x are places). A workgroup takes one tile of 16
// places x 64 outputs, 32 k at a time through LDS; float32 sums, k in order. With ff > 0 the weights hold
// [gate (ff) | up (ff)] rows and the kernel writes act[p, o] = g sigmoid(slope g) (u + shift), g = min(gate, limit),
// u = clamp(up, -limit, limit), o < ff, from both products.
template <typename T, typename TO, bool GLU>
__global__ void __launch_bounds__(256)
grouped_linear_kernel(const T* __restrict__ x, int ldx, const int* __restrict__ pair_at, int top, const T* __restrict__ w,
                      const int* __restrict__ offsets, const int* __restrict__ tiles, TO* __restrict__ out, int n_out, int K,
                      int ff, float limit, float slope, float shift) {
    __shared__ float xs[16][33], ws[64][33], wu[GLU ? 64 : 1][33];
    __shared__ int rows[16];
    const int e = tiles[2 * blockIdx.y];
    if (e < 0) return;
    const int p0 = tiles[2 * blockIdx.y + 1], pend = offsets[e + 1];
    const int o0 = blockIdx.x * 64;
    const int to = threadIdx.x % 64, tn = threadIdx.x / 64;
    if (threadIdx.x < 16) {
        const int p = p0 + threadIdx.x;
        rows[threadIdx.x] = p < pend ? (pair_at ? pair_at[p] / top : p) : -1;
    }
    __syncthreads();
    const int w_rows = GLU ? 2 * ff : n_out;
    const T* we = w + (size_t)e * w_rows * K;
    float acc[4] = {0.f, 0.f, 0.f, 0.f}, acu[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += 32) {
        for (int i = threadIdx.x; i < 16 * 32; i += 256) {
            const int rn = i / 32, rk = i % 32, r = rows[rn];
            xs[rn][rk] = (r >= 0 && k0 + rk < K) ? to_float(x[(size_t)r * ldx + k0 + rk]) : 0.f;
        }
        for (int i = threadIdx.x; i < 64 * 32; i += 256) {
            const int ro = i / 32, rk = i % 32;
            const bool in = o0 + ro < n_out && k0 + rk < K;
            ws[ro][rk] = in ? to_float(we[(size_t)(o0 + ro) * K + k0 + rk]) : 0.f;
            if (GLU) wu[ro][rk] = in ? to_float(we[(size_t)(ff + o0 + ro) * K + k0 + rk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 32; ++kk) {
            const float wv = ws[to][kk];
            const float uv = GLU ? wu[to][kk] : 0.f;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                acc[t] = fmaf(xs[tn * 4 + t][kk], wv, acc[t]);
                if (GLU) acu[t] = fmaf(xs[tn * 4 + t][kk], uv, acu[t]);
            }
        }
        __syncthreads();
    }
    if (o0 + to < n_out)
        for (int t = 0; t < 4; ++t) {
            const int p = p0 + tn * 4 + t;
            if (p >= pend) continue;
            float y = acc[t];
            if (GLU) {
                // gate and up are rounded as the compute dtype stores them before the activation
                const float g = fminf(to_float(from_float<T>(acc[t])), limit);
                const float u = fminf(fmaxf(to_float(from_float<T>(acu[t])), -limit), limit);
                y = g * hyb_sigmoid(slope * g) * (u + shift);
            }
            out[(size_t)p * n_out + o0 + to] = from_float<TO>(y);
        }
}

// The same products in bfloat16 on the matrix cores. A workgroup of four waves (WM x WN) takes a tile of
// BM = WM * MI * 16 places of one expert and BN = WN * NI * 16 weight rows, 64 k at a time through LDS, each wave
// MI x NI products of 16 x 16 x 32 with float32 sums; the places' rows of x are gathered while they are staged.
// With GLU a wave's weight tiles alternate between gate rows and the up rows of the same columns, so the
// activation is taken in registers and a workgroup writes BN / 2 columns of it.
typedef __attribute__((ext_vector_type(8))) __bf16 hyb_bf16x8;
typedef __attribute__((ext_vector_type(4))) float hyb_f32x4;
constexpr int GM_BK = 64, GM_STRIDE = GM_BK + 8;

template <int WM, int WN, int MI, int NI, bool GLU, typename TO>
__global__ void __launch_bounds__(256)
grouped_mfma_kernel(const bf16* __restrict__ x, int ldx, const int* __restrict__ pair_at, int top, const bf16* __restrict__ w,
                    const int* __restrict__ offsets, const int* __restrict__ tiles, TO* __restrict__ out, int n_out, int K, int ff,
                    float limit, float slope, float shift) {
    constexpr int BM = WM * MI * 16, BN = WN * NI * 16, COLS = GLU ? BN / 2 : BN;
    constexpr int A_PER = (BM * 8 + 255) / 256, W_PER = BN * 8 / 256;
    static_assert(WM * WN == 4 && (!GLU || NI % 2 == 0), "four waves; gate and up tiles in pairs");
    __shared__ __attribute__((aligned(16))) uint16_t As[2][BM * GM_STRIDE];     // two buffers: one barrier per 64 k
    __shared__ __attribute__((aligned(16))) uint16_t Ws[2][BN * GM_STRIDE];
    __shared__ int rows[BM];
    // (columns along x: workgroups that start together share a tile's rows of x. Measured the other way round,
    // tiles along x so that an expert's tiles share weight rows, a prompt of 2,048 tokens at 4B-sized layers took
    // 24.8 instead of 22.4 ms.)
    const int e = tiles[2 * blockIdx.y];
    if (e < 0) return;
    const int p0 = tiles[2 * blockIdx.y + 1], pend = offsets[e + 1];
    const int o0 = blockIdx.x * COLS;
    const int tid = threadIdx.x, wave = tid / SOC_WAVE, lane = tid % SOC_WAVE;
    const int wm = wave / WN, wn = wave % WN, li = lane % 16, lk = (lane / 16) * 8;
    for (int i = tid; i < BM; i += 256) {
        const int p = p0 + i;
        rows[i] = p < pend ? (pair_at ? pair_at[p] / top : p) : -1;
    }
    __syncthreads();
    const int w_rows = GLU ? 2 * ff : n_out;
    const bf16* we = w + (size_t)e * w_rows * K;
    // the weight row behind row r of the LDS tile (-1: none)
    auto weight_row = [&](int r) {
        if (!GLU) return o0 + r < n_out ? o0 + r : -1;
        const int rw = r / (NI * 16), j = (r % (NI * 16)) / 16, col = o0 + rw * (NI / 2 * 16) + (j / 2) * 16 + r % 16;
        return col < ff ? col + (j % 2 ? ff : 0) : -1;
    };
    const bf16* a_src[A_PER];
    const bf16* w_src[W_PER];
#pragma unroll
    for (int i = 0; i < A_PER; ++i) {
        const int c = tid + 256 * i, r = c < BM * 8 ? rows[c / 8] : -1;
        a_src[i] = r >= 0 ? x + (size_t)r * ldx + (c % 8) * 8 : nullptr;
    }
#pragma unroll
    for (int i = 0; i < W_PER; ++i) {
        const int c = tid + 256 * i, r = weight_row(c / 8);
        w_src[i] = r >= 0 ? we + (size_t)r * K + (c % 8) * 8 : nullptr;
    }
    hyb_f32x4 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = (hyb_f32x4){0.f, 0.f, 0.f, 0.f};
    uint4 ra[A_PER], rw[W_PER];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            const int kc = ((tid + 256 * i) % 8) * 8;
            ra[i] = (a_src[i] && k0 + kc < K) ? *reinterpret_cast<const uint4*>(a_src[i] + k0) : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int i = 0; i < W_PER; ++i) {
            const int kc = ((tid + 256 * i) % 8) * 8;
            rw[i] = (w_src[i] && k0 + kc < K) ? *reinterpret_cast<const uint4*>(w_src[i] + k0) : make_uint4(0u, 0u, 0u, 0u);
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            const int c = tid + 256 * i;
            if (c < BM * 8) *reinterpret_cast<uint4*>(&As[buf][(c / 8) * GM_STRIDE + (c % 8) * 8]) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < W_PER; ++i) {
            const int c = tid + 256 * i;
            *reinterpret_cast<uint4*>(&Ws[buf][(c / 8) * GM_STRIDE + (c % 8) * 8]) = rw[i];
        }
    };
    // blocks of 16 places of this wave that hold a place at all (the last tile of an expert is seldom full)
    const int n_sub = min(MI, max(0, (pend - p0 - wm * MI * 16 + 15) / 16));
    fetch(0);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += GM_BK, buf ^= 1) {
        const bool more = k0 + GM_BK < K;
        if (more) fetch(k0 + GM_BK);
#pragma unroll
        for (int ks = 0; ks < GM_BK; ks += 32) {
            hyb_bf16x8 wf[NI];
#pragma unroll
            for (int j = 0; j < NI; ++j)
                wf[j] = *reinterpret_cast<const hyb_bf16x8*>(&Ws[buf][((wn * NI + j) * 16 + li) * GM_STRIDE + ks + lk]);
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                if (i < n_sub) {                              // the same in all lanes of the wave
                    const hyb_bf16x8 af = *reinterpret_cast<const hyb_bf16x8*>(&As[buf][((wm * MI + i) * 16 + li) * GM_STRIDE + ks + lk]);
#pragma unroll
                    for (int j = 0; j < NI; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, wf[j], acc[i][j], 0, 0, 0);
                }
            }
        }
        // the other buffer was last read before the barrier that ended the previous round
        if (more) stash(buf ^ 1);
        __syncthreads();
    }
    // acc[i][j][r] belongs to place row 4 * (lane / 16) + r of tile i and weight row lane % 16 of tile j
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int p = p0 + (wm * MI + i) * 16 + (lane / 16) * 4 + r;
            if (p >= pend) continue;
            if constexpr (GLU) {
#pragma unroll
                for (int j = 0; j < NI; j += 2) {
                    const int col = o0 + wn * (NI / 2 * 16) + (j / 2) * 16 + li;
                    if (col >= ff) continue;
                    const float g = fminf(to_float(from_float<bf16>(acc[i][j][r])), limit);
                    const float u = fminf(fmaxf(to_float(from_float<bf16>(acc[i][j + 1][r])), -limit), limit);
                    out[(size_t)p * n_out + col] = from_float<TO>(g * hyb_sigmoid(slope * g) * (u + shift));
                }
            } else {
#pragma unroll
                for (int j = 0; j < NI; ++j) {
                    const int col = o0 + (wn * NI + j) * 16 + li;
                    if (col < n_out) out[(size_t)p * n_out + col] = from_float<TO>(acc[i][j][r]);
                }
            }
        }
}

// x [*, K]; w [E, 2 ff or n_out, K]; out [M, n_out] in the compute dtype (out_f32 0) or float32 (1). tile: the
// places per tile that the sorting kernel was given: 16 (any dtype; bfloat16 with K and ldx multiples of 8 on the
// matrix cores) or 128 (bfloat16 on the matrix cores only).
SOC_EXPORT int soc_grouped_linear(const void* x, int ldx, const int* pair_at, int top, const void* w, const int* offsets,
                                  const int* tiles, int max_tiles, int tile, void* out, int n_out, int K, int ff, float limit,
                                  float slope, float shift, int out_f32, int dtype, hipStream_t stream) {
    if (max_tiles <= 0 || n_out <= 0) return 0;
    if (K < 1 || max_tiles > 65535 || (ff > 0 && (ff != n_out || out_f32))) return (int)hipErrorInvalidValue;
    const bool mfma = dtype == 1 && K % 8 == 0 && ldx % 8 == 0;
    if ((tile != 16 && tile != 128) || (tile > 16 && !mfma)) return (int)hipErrorInvalidValue;
    if (mfma) {
#define SOC_GM(WM, WN, MI, NI, GLU, TO)                                                                                          \
    hipLaunchKernelGGL((grouped_mfma_kernel<WM, WN, MI, NI, GLU, TO>), dim3((n_out + (GLU ? 63 : 127)) / (GLU ? 64 : 128), max_tiles), \
                       dim3(256), 0, stream, (const bf16*)x, ldx, pair_at, top, (const bf16*)w, offsets, tiles, (TO*)out, n_out, \
                       K, ff, limit, slope, shift)
        if (tile == 128) {
            if (ff > 0) SOC_GM(2, 2, 4, 4, true, bf16); else if (out_f32) SOC_GM(2, 2, 4, 4, false, float); else SOC_GM(2, 2, 4, 4, false, bf16);
        } else {
            if (ff > 0) SOC_GM(1, 4, 1, 2, true, bf16); else if (out_f32) SOC_GM(1, 4, 1, 2, false, float); else SOC_GM(1, 4, 1, 2, false, bf16);
        }
#undef SOC_GM
        return soc_last_error();
    }
    const dim3 grid((n_out + 63) / 64, max_tiles);
#define SOC_GL(T, TO, GLU)                                                                                                    \
    hipLaunchKernelGGL((grouped_linear_kernel<T, TO, GLU>), grid, dim3(256), 0, stream, (const T*)x, ldx, pair_at, top,       \
                       (const T*)w, offsets, tiles, (TO*)out, n_out, K, ff, limit, slope, shift)
    if (ff > 0) { if (dtype == 0) SOC_GL(float, float, true); else SOC_GL(bf16, bf16, true); }
    else if (dtype == 0) SOC_GL(float, float, false);
    else if (out_f32) SOC_GL(bf16, float, false);
    else SOC_GL(bf16, bf16, false);
#undef SOC_GL
    return soc_last_error();
}

// ---- the weighted sum of a token's experts ---------------------------------------------------------------------------
// out[n, c] = sum_r weight[n, r] y[place[n top + r], c] (+ extra[n, c], times sigmoid(gate[n ldg]) if gate is given), float32;
// y float32 [M, d] by place.
template <typename T>
__global__ void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ place, const float* __restrict__ weight,
                                   const T* __restrict__ extra, const float* __restrict__ gate, int ldg, float* __restrict__ out,
                                   int N, int d, int top) {
    const int n = blockIdx.y;
    const float open = (extra && gate) ? hyb_sigmoid(gate[(size_t)n * ldg]) : 1.f;
    for (int c = blockIdx.x * blockDim.x + threadIdx.x; c < d; c += gridDim.x * blockDim.x) {
        float acc = extra ? open * to_float(extra[(size_t)n * d + c]) : 0.f;
        for (int r = 0; r < top; ++r)
            acc = fmaf(weight[(size_t)n * top + r], y[(size_t)place[(size_t)n * top + r] * d + c], acc);
        out[(size_t)n * d + c] = acc;
    }
}

SOC_EXPORT int soc_moe_combine(const float* y, const int* place, const float* weight, const void* extra, const float* gate, int ldg,
                               float* out, int N, int d, int top, int dtype, hipStream_t stream) {
    if (N <= 0 || d <= 0) return 0;
    if (N > 65535) return (int)hipErrorInvalidValue;
    const dim3 grid((d + 255) / 256 < 16 ? (d + 255) / 256 : 16, N);
    if (dtype == 0)
        hipLaunchKernelGGL(moe_combine_kernel<float>, grid, dim3(256), 0, stream, y, place, weight, (const float*)extra, gate, ldg, out, N, d, top);
    else
        hipLaunchKernelGGL(moe_combine_kernel<bf16>, grid, dim3(256), 0, stream, y, place, weight, (const bf16*)extra, gate, ldg, out, N, d, top);
    return soc_last_error();
}

// ---- a per-token side input: gelu_tanh(t) * table[token, col0 + j] -----------------------------------------------------
template <typename T>
__global__ void side_gate_kernel(const T* __restrict__ t, const T* __restrict__ table, int ldt, int col0, const int* __restrict__ ids,
                                 int V, T* __restrict__ out, size_t total, int dim) {
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const size_t n = e / dim;
        const int j = (int)(e % dim);
        const int id = min(max(ids[n], 0), V - 1);
        const float z = to_float(t[e]);
        const float g = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
        out[e] = from_float<T>(g * to_float(table[(size_t)id * ldt + col0 + j]));
    }
}

SOC_EXPORT int soc_side_gate(const void* t, const void* table, int ldt, int col0, const int* ids, int V, void* out, int N, int dim,
                             int dtype, hipStream_t stream) {
    const size_t total = (size_t)N * dim;
    if (!total) return 0;
    if (col0 < 0 || col0 + dim > ldt || V < 1) return (int)hipErrorInvalidValue;
    const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    if (dtype == 0)
        hipLaunchKernelGGL(side_gate_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)t, (const float*)table, ldt, col0,
                           ids, V, (float*)out, total, dim);
    else
        hipLaunchKernelGGL(side_gate_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)t, (const bf16*)table, ldt, col0,
                           ids, V, (bf16*)out, total, dim);
    return soc_last_error();
}

// ---- residual += delta, and the sum in the compute dtype ---------------------------------------------------------------
// delta: nothing, [N, d] in the compute dtype, or float32 partial sums [S, N, d] added in order.
template <typename T>
__global__ void add_cast_kernel(float* __restrict__ residual, const T* __restrict__ whole, const float* __restrict__ parts,
                                int n_parts, size_t total, T* __restrict__ out) {
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        float r = residual[e];
        if (whole) r += to_float(whole[e]);
        for (int s = 0; s < n_parts; ++s) r += parts[(size_t)s * total + e];
        if (whole || n_parts) residual[e] = r;
        out[e] = from_float<T>(r);
    }
}

SOC_EXPORT int soc_add_cast(float* residual, const void* whole, const float* parts, int n_parts, long long total, void* out,
                            int dtype, hipStream_t stream) {
    if (total <= 0) return 0;
    const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
    if (dtype == 0)
        hipLaunchKernelGGL(add_cast_kernel<float>, dim3(blocks), dim3(256), 0, stream, residual, (const float*)whole, parts, n_parts,
                           (size_t)total, (float*)out);
    else
        hipLaunchKernelGGL(add_cast_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, residual, (const bf16*)whole, parts, n_parts,
                           (size_t)total, (bf16*)out);
    return soc_last_error();
}
