// Kernels of a matrix memory with exponential gates (the gates with their running maximum, what they make of
// q, k and the decays ahead of the recurrence, and the denominators, head norms and gate behind it), and of
// differential attention (the second map subtracted from the first, the head's norm).
//
// Gates, their logarithms and exponentials, the running maximum, denominators and norms' statistics are float32
// whatever the compute dtype; a value is rounded once, where it is stored in the compute dtype.
#include "common.h"

__device__ __forceinline__ float mem_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }
// log(sigmoid(u)) = min(u, 0) - log(1 + exp(-|u|))
__device__ __forceinline__ float mem_logsigmoid(float u) { return fminf(u, 0.f) - log1pf(expf(-fabsf(u))); }

// ---- the gates of a step's tokens and their running maximum --------------------------------------------------------
// gates: float32 [N, 2 H], the logits of the input gates (columns 0 .. H - 1) and of the forget gates (H .. 2 H - 1);
// bias float32 [2 H]. i = cap tanh((z_i + b_i) / cap), f = logsigmoid(cap tanh((z_f + b_f) / cap)). Per sequence and
// head, from the maximum m that the row's state holds (at offset + head): m' = max(f + m, i), keep = exp(f + m - m'),
// take = exp(i - m'); maxima, keep and take are float32 [N, H]; the row's maximum is left for the next step. A token is
// the map m -> max(F + m, I) with (F, I) = (f, i), and maps compose as (F1, I1) then (F2, I2) = (F1 + F2, max(I1 + F2,
// I2)). One workgroup per (sequence, head), of 1 to 16 waves (more for long portions), walks blockDim.x tokens per
// round: every wave composes its 64 tokens' maps in order by a scan over its lanes, the waves' totals meet in LDS,
// and a token's maximum is the map of all tokens of the round before it applied to what the rounds before left.
struct GateMap { float F, I; };
__device__ __forceinline__ GateMap then(GateMap a, GateMap b) { return GateMap{a.F + b.F, fmaxf(a.I + b.F, b.I)}; }

__global__ void __launch_bounds__(1024)
memory_scan_kernel(const float* __restrict__ gates, const float* __restrict__ bias, float cap, int H,
                   float* __restrict__ state, size_t stride, int offset, const int* __restrict__ seq_qstart,
                   const int* __restrict__ seq_rows, float* __restrict__ maxima, float* __restrict__ keep,
                   float* __restrict__ take) {
    __shared__ float totals[2][16][2];
    const int seq = blockIdx.y, head = blockIdx.x;
    const int wave = threadIdx.x / SOC_WAVE, lane = threadIdx.x % SOC_WAVE, n_waves = blockDim.x / SOC_WAVE;
    const int lo = seq_qstart[seq], hi = seq_qstart[seq + 1];
    if (lo >= hi) return;                                   // (the whole workgroup: no barrier is left waiting)
    float* held = state + (size_t)seq_rows[seq] * stride + offset + head;
    float carry = *held;
    const float bi = bias[head], bf = bias[H + head], inv_cap = 1.f / cap;
    int buf = 0;
    for (int n0 = lo; n0 < hi; n0 += blockDim.x, buf ^= 1) {
        const int n = n0 + threadIdx.x;
        const bool in = n < hi;
        float gi = -INFINITY, gf = 0.f;                    // (behind the end: the map that changes nothing)
        if (in) {
            gi = cap * tanhf((gates[(size_t)n * 2 * H + head] + bi) * inv_cap);
            gf = mem_logsigmoid(cap * tanhf((gates[(size_t)n * 2 * H + H + head] + bf) * inv_cap));
        }
        GateMap mine{gf, gi};                               // becomes the map of the wave's tokens up to this one
#pragma unroll
        for (int d = 1; d < SOC_WAVE; d <<= 1) {
            const GateMap before{__shfl_up(mine.F, d, SOC_WAVE), __shfl_up(mine.I, d, SOC_WAVE)};
            if (lane >= d) mine = then(before, mine);
        }
        if (lane == SOC_WAVE - 1) { totals[buf][wave][0] = mine.F; totals[buf][wave][1] = mine.I; }
        __syncthreads();
        GateMap ahead{0.f, -INFINITY}, whole{0.f, -INFINITY};     // the waves before this one; all waves of the round
        for (int w = 0; w < n_waves; ++w) {
            const GateMap t{totals[buf][w][0], totals[buf][w][1]};
            if (w < wave) ahead = then(ahead, t);
            whole = then(whole, t);
        }
        const float start = fmaxf(ahead.F + carry, ahead.I);      // the maximum in front of this wave's first token
        const float m = fmaxf(mine.F + start, mine.I);
        float before = __shfl_up(m, 1, SOC_WAVE);
        if (lane == 0) before = start;
        if (in) {
            maxima[(size_t)n * H + head] = m;
            keep[(size_t)n * H + head] = expf(gf + before - m);
            take[(size_t)n * H + head] = expf(gi - m);
        }
        carry = fmaxf(whole.F + carry, whole.I);
    }
    if (threadIdx.x == 0) *held = carry;
}

// prep [N, 3, H D] float32: q scaled, k times the token's take, and the token's keep for every key channel.
template <typename T>
__global__ void memory_prepare_kernel(const T* __restrict__ x, int ld, int col_q, int col_k, float q_scale,
                                      const float* __restrict__ keep, const float* __restrict__ take, int H, int D,
                                      size_t total, float* __restrict__ prep) {
    const int HD = H * D;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
        const int c = (int)(e % HD);
        const size_t n = e / HD;
        const int h = c / D;
        float* row = prep + n * 3 * HD + c;
        row[0] = to_float(x[n * ld + col_q + c]) * q_scale;
        row[HD] = to_float(x[n * ld + col_k + c]) * take[n * H + h];
        row[2 * (size_t)HD] = keep[n * H + h];
    }
}

SOC_EXPORT int soc_memory_gates(const float* gates, const float* bias, float cap, const void* x, int ld, int col_q, int col_k,
                                float q_scale, int H, int D, float* state, long long stride, int offset,
                                const int* seq_qstart, const int* seq_rows, int n_seqs, int max_q_len, int N, float* maxima,
                                float* keep, float* take, float* prep, int dtype, hipStream_t stream) {
    if (n_seqs <= 0 || N <= 0 || H <= 0) return 0;
    if (D < 1 || !(cap > 0.f) || n_seqs > 65535 || offset < 0) return (int)hipErrorInvalidValue;
    // waves per (sequence, head): one for single tokens and short portions, up to sixteen for long ones
    const int threads = max_q_len <= 64 ? 64 : max_q_len <= 256 ? 256 : 1024;
    hipLaunchKernelGGL(memory_scan_kernel, dim3(H, n_seqs), dim3(threads), 0, stream, gates, bias, cap, H, state, (size_t)stride,
                       offset, seq_qstart, seq_rows, maxima, keep, take);
    const size_t total = (size_t)N * H * D;
    const int blocks = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
    if (dtype == 0)
        hipLaunchKernelGGL(memory_prepare_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)x, ld, col_q, col_k,
                           q_scale, keep, take, H, D, total, prep);
    else
        hipLaunchKernelGGL(memory_prepare_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)x, ld, col_q, col_k,
                           q_scale, keep, take, H, D, total, prep);
    return soc_last_error();
}

// ---- behind the recurrence: denominators, head norms, gain and gate ----------------------------------------------------
// raw: float32 [N, H, Dv + 1], a head's S^T q and, last, n . q. o = raw[.. Dv] / (max(|n . q|, exp(-m)) + den_eps) with
// m = maxima[n, h]; o over its root mean square (eps inside the root), times gain [H Dv], times sigmoid(z[n, h Dv + c])
// (z: rows of ldz elements in the compute dtype). One wave per (token, head).
template <typename T>
__global__ void __launch_bounds__(256)
memory_finish_kernel(const float* __restrict__ raw, const float* __restrict__ maxima, const T* __restrict__ z, int ldz,
                     const float* __restrict__ gain, int H, int Dv, float eps, float den_eps, size_t items,
                     T* __restrict__ out) {
    const int wave = threadIdx.x / SOC_WAVE, lane = threadIdx.x % SOC_WAVE;
    const size_t item = (size_t)blockIdx.x * 4 + wave;
    if (item >= items) return;
    const size_t n = item / H;
    const int h = (int)(item % H);
    const float* row = raw + item * (Dv + 1);
    const float den = fmaxf(fabsf(row[Dv]), expf(-maxima[item])) + den_eps;
    float ss = 0.f;
    for (int c = lane; c < Dv; c += SOC_WAVE) { const float o = row[c] / den; ss = fmaf(o, o, ss); }
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float)Dv + eps);
    for (int c = lane; c < Dv; c += SOC_WAVE) {
        const int col = h * Dv + c;
        out[n * H * Dv + col] = from_float<T>(row[c] / den * inv * gain[col] * mem_sigmoid(to_float(z[n * ldz + col])));
    }
}

SOC_EXPORT int soc_memory_finish(const float* raw, const float* maxima, const void* z, int ldz, const float* gain, int N, int H,
                                 int Dv, float eps, float den_eps, void* out, int dtype, hipStream_t stream) {
    const size_t items = (size_t)N * H;
    if (!items) return 0;
    if (Dv < 1 || ldz < H * Dv || (items + 3) / 4 > 0x7fffffff) return (int)hipErrorInvalidValue;
    const dim3 grid((unsigned)((items + 3) / 4));
    if (dtype == 0)
        hipLaunchKernelGGL(memory_finish_kernel<float>, grid, dim3(256), 0, stream, raw, maxima, (const float*)z, ldz, gain, H, Dv,
                           eps, den_eps, items, (float*)out);
    else
        hipLaunchKernelGGL(memory_finish_kernel<bf16>, grid, dim3(256), 0, stream, raw, maxima, (const bf16*)z, ldz, gain, H, Dv,
                           eps, den_eps, items, (bf16*)out);
    return soc_last_error();
}

// ---- differential attention: a head's two maps combined ----------------------------------------------------------------
// o: [N, 2 H, P], the attention results laid out (kv head g, map, query head r of the group): head h = g R + r has its
// first map at (2 g) R + r and its second at (2 g + 1) R + r, R = H / G. y = a1 - lam a2 over the first Dv elements,
// over its root mean square (eps inside the root), times out_scale: out [N, H Dv]. One wave per (token, head).
template <typename T>
__global__ void __launch_bounds__(256)
diff_combine_kernel(const T* __restrict__ o, int H, int R, int P, int Dv, float lam, float eps, float out_scale, size_t items,
                    T* __restrict__ out) {
    const int wave = threadIdx.x / SOC_WAVE, lane = threadIdx.x % SOC_WAVE;
    const size_t item = (size_t)blockIdx.x * 4 + wave;
    if (item >= items) return;
    const size_t n = item / H;
    const int h = (int)(item % H), g = h / R, r = h % R;
    const T* a1 = o + (n * 2 * H + (size_t)(2 * g) * R + r) * P;
    const T* a2 = o + (n * 2 * H + (size_t)(2 * g + 1) * R + r) * P;
    float ss = 0.f;
    for (int c = lane; c < Dv; c += SOC_WAVE) { const float y = to_float(a1[c]) - lam * to_float(a2[c]); ss = fmaf(y, y, ss); }
    const float inv = out_scale / sqrtf(wave_sum(ss) / (float)Dv + eps);
    for (int c = lane; c < Dv; c += SOC_WAVE)
        out[item * Dv + c] = from_float<T>((to_float(a1[c]) - lam * to_float(a2[c])) * inv);
}

SOC_EXPORT int soc_diff_combine(const void* o, void* out, int N, int H, int G, int P, int Dv, float lam, float eps, float out_scale,
                                int dtype, hipStream_t stream) {
    const size_t items = (size_t)N * H;
    if (!items) return 0;
    if (G < 1 || H % G || Dv < 1 || Dv > P || (items + 3) / 4 > 0x7fffffff) return (int)hipErrorInvalidValue;
    const dim3 grid((unsigned)((items + 3) / 4));
    if (dtype == 0)
        hipLaunchKernelGGL(diff_combine_kernel<float>, grid, dim3(256), 0, stream, (const float*)o, H, H / G, P, Dv, lam, eps, out_scale,
                           items, (float*)out);
    else
        hipLaunchKernelGGL(diff_combine_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)o, H, H / G, P, Dv, lam, eps, out_scale,
                           items, (bf16*)out);
    return soc_last_error();
}
