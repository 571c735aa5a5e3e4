// Sequence-mixing kernels for hybrid models (gfx950): bias-free LayerNorm and
// RMS norms on an fp32 residual stream (with the post-norm residual step fused),
// short causal convolutions with a carried tail, paged KV scatter with distinct
// K/V head sizes, interleaved rotary positions, paged softmax attention with
// optional sliding window / always-visible first tokens / log-distance penalty /
// query temperature / tanh score cap / softmax sink, the gated delta-rule
// linear recurrence, and gated feed-forward activations.
//
// Built as a plain C-ABI shared library (no torch headers): the Python side
// passes raw device pointers and the current HIP stream, so the kernels are
// stream-ordered with the surrounding torch ops and hipGraph-capturable.
//
// Step layout shared by all kernels: activations are (B, S, ...) row-major;
// `pos` (B,S) int32 holds each token's position or -1 for padding; the real
// tokens of a row sit at columns 0..n-1 with consecutive positions; `seq`
// (B) int32 is the row's state slot or -1; `nvalid` (B) int32 is n.
// Statistics, scores, softmax, decays and the recurrent state are fp32
// regardless of the activation type.

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#define WAVE 64
#define DEV __device__ __forceinline__

typedef __hip_bfloat16 bf16;

template <typename T> DEV float ldf(const T* p);
template <> DEV float ldf<float>(const float* p) { return *p; }
template <> DEV float ldf<bf16>(const bf16* p) { return __bfloat162float(*p); }
template <typename T> DEV void stf(T* p, float v);
template <> DEV void stf<float>(float* p, float v) { *p = v; }
template <> DEV void stf<bf16>(bf16* p, float v) { *p = __float2bfloat16(v); }

DEV float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
DEV float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}
DEV float sigmoidf_(float x) { return 1.f / (1.f + expf(-x)); }
DEV float softplusf_(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// 8 consecutive elements as floats, one or two 16-byte loads
template <typename T> DEV void load8(const T* p, float* v);
template <> DEV void load8<bf16>(const bf16* p, float* v) {
    const uint4 raw = *reinterpret_cast<const uint4*>(p);
    const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        v[2 * e] = __uint_as_float(u[e] << 16);
        v[2 * e + 1] = __uint_as_float(u[e] & 0xffff0000u);
    }
}
template <> DEV void load8<float>(const float* p, float* v) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}


// ---------------------------------------------------------------- LayerNorm
// one 256-thread workgroup per row; mean, then variance of the deviations
// (both fp32); the row is re-read from cache, not kept in registers, so any
// width works
#define LN_THREADS 256

DEV float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & (WAVE - 1), wv = threadIdx.x / WAVE;
    __syncthreads();                       // red may still be read by the previous call
    if (lane == 0) red[wv] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < LN_THREADS / WAVE; ++i) t += red[i];
    return t;
}

template <typename TOut>
__global__ void __launch_bounds__(LN_THREADS)
layer_norm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                  TOut* __restrict__ out, long rows, int C, float eps) {
    __shared__ float red[LN_THREADS / WAVE];
    const long row = blockIdx.x;
    const float* xr = x + row * C;
    float s = 0.f;
    for (int c = threadIdx.x; c < C; c += LN_THREADS) s += xr[c];
    const float mean = block_sum(s, red) / C;
    float v = 0.f;
    for (int c = threadIdx.x; c < C; c += LN_THREADS) { float d = xr[c] - mean; v += d * d; }
    const float inv = 1.f / sqrtf(block_sum(v, red) / C + eps);
    TOut* o = out + row * C;
    for (int c = threadIdx.x; c < C; c += LN_THREADS) stf<TOut>(o + c, (xr[c] - mean) * inv * w[c]);
}

// ------------------------------------------------------------- short conv
// y[b,t,c] = act(sum_j w[c,j] * x[b, t-R+j, c]) (+ x[b,t,c]); columns before
// the step come from the carried tail (oldest first), positions < 0 are zero
// y[b,t,c] = act(sum_j w[c,j] * x[b, t-R+j, c]) (+ x[b,t,c]); columns before
// the step come from the carried tail (oldest first), positions < 0 are zero.
// `xs` is the input's row stride in elements (a column slice of a wider
// projection is read in place); y is dense. One thread per element: adjacent
// lanes read adjacent channels of the same row for every tap.
template <typename TIn, typename TOut>
__global__ void short_conv_kernel(const TIn* __restrict__ x, long xs, const float* __restrict__ w,
                                  const float* __restrict__ tail, const int* __restrict__ pos,
                                  const int* __restrict__ seq, TOut* __restrict__ y,
                                  int B, int S, int C, int taps, int act_silu, int residual,
                                  const float* __restrict__ bias) {
    const long total = (long)B * S * C;
    const int R = taps - 1;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int c = idx % C;
        const long bt = idx / C;
        const int t = bt % S;
        const int b = bt / S;
        const int p = pos[bt];
        const int slot = seq[b];
        if (p < 0 || slot < 0) { stf<TOut>(y + idx, 0.f); continue; }
        const float* wr = w + (long)c * taps;
        float acc = bias ? bias[c] : 0.f, cur = 0.f;
        for (int j = 0; j < taps; ++j) {
            const int col = t - R + j;
            float xv;
            if (col >= 0) {
                xv = ldf<TIn>(x + ((long)b * S + col) * xs + c);
            } else {
                const int ps = p - R + j;              // source position
                xv = ps < 0 ? 0.f : tail[((long)slot * R + (R + col)) * C + c];
            }
            acc += wr[j] * xv;
            cur = xv;
        }
        if (act_silu) acc = acc * sigmoidf_(acc);
        if (residual) acc += cur;
        stf<TOut>(y + idx, acc);
    }
}

// Tiled variant for the common filter lengths: a thread owns 8 adjacent
// channels, keeps their taps in registers and walks SC_TT consecutive tokens
// with a sliding window of the last TAPS-1 inputs, so every input element is
// loaded once (16 bytes per load) instead of TAPS times.
#define SC_TT 16

template <typename T> DEV void st8(T* p, const float* v);
template <> DEV void st8<float>(float* p, const float* v) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}

template <typename TIn, typename TOut, int TAPS>
__global__ void short_conv_tile_kernel(const TIn* __restrict__ x, long xs,
                                       const float* __restrict__ w,
                                       const float* __restrict__ tail,
                                       const int* __restrict__ pos, const int* __restrict__ seq,
                                       const int* __restrict__ nvalid, TOut* __restrict__ y,
                                       int S, int C, int tiles_per_row, int act_silu,
                                       int residual, const float* __restrict__ bias) {
    constexpr int R = TAPS - 1;
    const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (c >= C) return;
    const int b = blockIdx.y / tiles_per_row;
    const int t0 = (blockIdx.y % tiles_per_row) * SC_TT;
    const int t1 = min(t0 + SC_TT, S);
    const int slot = seq[b];
    const int n = slot < 0 ? 0 : nvalid[b];
    const int p0 = pos[(long)b * S];
    float wr[8][TAPS];
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
        for (int j = 0; j < TAPS; ++j) wr[e][j] = w[(long)(c + e) * TAPS + j];
    float bs[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) bs[e] = bias ? bias[c + e] : 0.f;
    float hist[R > 0 ? R : 1][8];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int col = t0 - R + r;
        if (col >= 0) {
            load8<TIn>(x + ((long)b * S + col) * xs + c, hist[r]);
        } else {
            const float* tp = tail + ((long)(slot < 0 ? 0 : slot) * R + (R + col)) * C + c;
#pragma unroll
            for (int e = 0; e < 8; ++e) hist[r][e] = (n > 0 && p0 + col >= 0) ? tp[e] : 0.f;
        }
    }
    for (int t = t0; t < t1; ++t) {
        float o[8];
        if (t < n) {
            float cur[8];
            load8<TIn>(x + ((long)b * S + t) * xs + c, cur);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float acc = bs[e];
#pragma unroll
                for (int r = 0; r < R; ++r) acc += wr[e][r] * hist[r][e];
                acc += wr[e][R] * cur[e];
                if (act_silu) acc = acc * sigmoidf_(acc);
                if (residual) acc += cur[e];
                o[e] = acc;
            }
#pragma unroll
            for (int r = 0; r + 1 < R; ++r)
#pragma unroll
                for (int e = 0; e < 8; ++e) hist[r][e] = hist[r + 1][e];
            if (R > 0) {
#pragma unroll
                for (int e = 0; e < 8; ++e) hist[R - 1][e] = cur[e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = 0.f;
        }
        TOut* yp = y + ((long)b * S + t) * C + c;
        if constexpr (sizeof(TOut) == 2) {
            uint32_t pk[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                uint32_t lo = __float_as_uint(o[2 * e]), hi = __float_as_uint(o[2 * e + 1]);
                lo += 0x7fffu + ((lo >> 16) & 1u);
                hi += 0x7fffu + ((hi >> 16) & 1u);
                pk[e] = (lo >> 16) | (hi & 0xffff0000u);
            }
            *reinterpret_cast<uint4*>(yp) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
        } else {
            st8<float>(reinterpret_cast<float*>(yp), o);
        }
    }
}

// new tail = last R inputs of (old tail ++ this step's inputs); one thread per
// (row, channel) so the in-place shift is private to the thread
template <typename TIn>
__global__ void short_conv_commit_kernel(const TIn* __restrict__ x, long xs,
                                         float* __restrict__ tail,
                                         const int* __restrict__ pos, const int* __restrict__ seq,
                                         const int* __restrict__ nvalid, int B, int S, int C, int R) {
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)B * C) return;
    const int c = idx % C;
    const int b = idx / C;
    const int slot = seq[b];
    const int n = nvalid[b];
    if (slot < 0 || n <= 0) return;
    const int p0 = pos[(long)b * S];
    float* tr = tail + (long)slot * R * C + c;
    for (int r = 0; r < R; ++r) {
        const int col = n - R + r;
        float v;
        if (col >= 0) v = ldf<TIn>(x + ((long)b * S + col) * xs + c);
        else v = (p0 + col) < 0 ? 0.f : tr[(long)(R + col) * C];
        tr[(long)r * C] = v;
    }
}

// ------------------------------------------------------------ paged KV write
template <typename T>
__global__ void paged_kv_write_kernel(T* __restrict__ kc, T* __restrict__ vc,
                                      const T* __restrict__ k, long kstride,
                                      const T* __restrict__ v, long vstride,
                                      const int* __restrict__ slots, long N, int GDk, int GDv,
                                      long nslots) {
    const int per = GDk + GDv;
    const long total = N * per;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const long tok = idx / per;
        const int e = idx % per;
        const int s = slots[tok];
        if (s < 0 || s >= nslots) continue;
        if (e < GDk) kc[(long)s * GDk + e] = k[tok * kstride + e];
        else vc[(long)s * GDv + (e - GDk)] = v[tok * vstride + (e - GDk)];   // GDv = 0: no V
    }
}

// --------------------------------------------- latent cache row, one launch
// A latent layer's cache row of a token: [rms_norm(x[:C]) * w | x[C:C+R] with its
// first 2*half channels turned in interleaved pairs by pos * inv_freq[i]], written
// straight into the token's page slot (and, when `row` is given, into a dense row
// buffer as well). One wave per token; statistics and angles in fp32. Pad tokens
// (slot or position < 0) write nothing to the cache.
template <typename T>
__global__ void latent_row_kernel(const T* __restrict__ x, long xs, const float* __restrict__ w,
                                  float eps, const float* __restrict__ inv_freq, int half,
                                  const int* __restrict__ pos, const int* __restrict__ slots,
                                  T* __restrict__ cache, long nslots, T* __restrict__ row, long rs,
                                  long ntok, int C, int R) {
    const int lane = threadIdx.x & (WAVE - 1);
    const long tok = (long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (tok >= ntok) return;
    const int s = slots[tok], p = pos[tok];
    T* cp = (s >= 0 && s < nslots && p >= 0) ? cache + (long)s * (C + R) : nullptr;
    T* rp = row ? row + tok * rs : nullptr;
    if (!cp && !rp) return;
    const T* xr = x + tok * xs;
    float ss = 0.f;
    for (int c = lane; c < C; c += WAVE) { const float v = ldf<T>(xr + c); ss += v * v; }
    const float inv = 1.f / sqrtf(wave_sum(ss) / C + eps);
    for (int c = lane; c < C; c += WAVE) {
        const float v = ldf<T>(xr + c) * inv * w[c];
        if (cp) stf<T>(cp + c, v);
        if (rp) stf<T>(rp + c, v);
    }
    for (int e = lane; e < half + (R - 2 * half); e += WAVE) {
        if (e < half) {
            const float a = ldf<T>(xr + C + 2 * e), b = ldf<T>(xr + C + 2 * e + 1);
            float sn, cs;
            sincosf((float)(p < 0 ? 0 : p) * inv_freq[e], &sn, &cs);
            const float u = a * cs - b * sn, v = b * cs + a * sn;
            if (cp) { stf<T>(cp + C + 2 * e, u); stf<T>(cp + C + 2 * e + 1, v); }
            if (rp) { stf<T>(rp + C + 2 * e, u); stf<T>(rp + C + 2 * e + 1, v); }
        } else {
            const int c = C + 2 * half + (e - half);
            const float v = ldf<T>(xr + c);
            if (cp) stf<T>(cp + c, v);
            if (rp) stf<T>(rp + c, v);
        }
    }
}

// ----------------------------------------------------------- paged attention
// Score of query i and key j, in order: q.k * scale * temp(i), temp(i) = 1 +
// qt_coef * ln(floor((i+1)/qt_every) + 1) (qt_every = 0: none); minus
// r1_h * log(1 + r2_h (i-j)) (r1 = null: none); cap * tanh(. / cap) (cap = 0:
// none); a lone r1 (r2 = null) is a linear penalty r1_h * (i-j) instead.
// Visible: j <= i and (i-j < window or j < keep); plain causal attention
// passes window = INT_MAX. With cmask > 0 also only keys of the query's own block
// of cmask positions (j >= floor(i/cmask)*cmask). `sink` (per head, or null)
// adds exp(sink_h) to the softmax denominator. K and V rows are addressed as slot*tok_stride +
// head*head_stride, so V may be a channel range of the K rows.
// Workgroup (4 waves) = ATT_NQ query rows that share one KV head: HPW query
// heads of the group x QT consecutive tokens of a batch row, so every K/V
// line fetched serves all of them. The union of the rows' visible keys is
// [0, min(keep, lo)) + [lo, i_max], lo = the larger of max(0, i_min-window+1)
// and i_min's block start; each row masks by its own position. Waves
// take 64-key tiles round-robin: a lane owns one key for the scores (q rows
// broadcast from LDS, fp32 accumulate, online softmax per row), then the
// wave's P tile goes through LDS and a lane owns value channels for P.V.
// The four partial results merge through LDS at the end. One kernel serves
// prompt portions, decoded tokens and mixed batches.
// Two shapes: (NQ=16 rows, 4 waves) for steps with prompt portions, and
// (NQ=4 rows, 16 waves) for pure decode steps, where one token's few heads
// leave the key range as the only parallelism.
#define ATT_NQ_MAX 16

template <typename T, typename TOut, int MAXR, int ATT_NQ, int ATT_WAVES>
__global__ void __launch_bounds__(ATT_WAVES * WAVE)
window_attn_kernel(const T* __restrict__ q, long qstride, const T* __restrict__ kc,
                   const T* __restrict__ vc, const int* __restrict__ pos,
                   const int* __restrict__ seq,
                   const int* __restrict__ btab, int max_blocks, const float* __restrict__ r1,
                   const float* __restrict__ r2, const T* __restrict__ gate, long gstride,
                   TOut* __restrict__ out, int H, int G, int Dk, int Dv,
                   int bsz, int S, float scale, int window, int keep, int HPW, int QT,
                   int chunks, int lpr, int pws, long ktok, long khead, long vtok, long vhead,
                   int kvec, const float* __restrict__ sink, float cap, float qt_coef,
                   int qt_every, int ghead, int cmask) {
    // lpr > 0 (decode shape only): P.V with 8 value channels per lane and
    // 64/lpr keys per step, 16-byte V loads; pws = floats of LDS per wave
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int DkP = (Dk + 7) & ~7;                       // padded q row
    float* qs = smem;                                    // ATT_NQ * DkP
    float* ps = qs + ATT_NQ * DkP;                       // ATT_WAVES * 64 * ATT_NQ
    float* cs = ps;                                      // merge area reuses the P tiles
    constexpr int ATT_THREADS = ATT_WAVES * WAVE;
    __shared__ int rpos[ATT_NQ_MAX], rclo[ATT_NQ_MAX];
    __shared__ float ra1[ATT_NQ_MAX], ra2[ATT_NQ_MAX], rtemp[ATT_NQ_MAX], rsink[ATT_NQ_MAX];

    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wv = tid / WAVE;
    const int b = blockIdx.z;
    const int g = blockIdx.y / chunks, chunk = blockIdx.y % chunks;
    const int t0 = blockIdx.x * QT;
    const int rep = H / G;
    if (seq[b] < 0) return;
    // row table
    if (tid < ATT_NQ) {
        const int tq = tid / HPW, hh = chunk * HPW + tid % HPW;
        int p = -1;
        if (tq < QT && t0 + tq < S && hh < rep) p = pos[(long)b * S + t0 + tq];
        rpos[tid] = p;
        rclo[tid] = (cmask > 0 && p >= 0) ? (p / cmask) * cmask : 0;
        const int h = g * rep + (hh < rep ? hh : 0);
        ra1[tid] = r1 ? r1[h] : 0.f;
        ra2[tid] = r2 ? r2[h] : 0.f;
        rsink[tid] = sink ? sink[h] : -INFINITY;
        rtemp[tid] = (qt_every > 0 && p >= 0)
            ? 1.f + qt_coef * logf((float)((p + 1) / qt_every) + 1.f) : 1.f;
    }
    __syncthreads();
    int i_min = 0x7fffffff, i_max = -1;
#pragma unroll
    for (int r = 0; r < ATT_NQ; ++r) {
        const int p = rpos[r];
        if (p >= 0) { i_min = min(i_min, p); i_max = max(i_max, p); }
    }
    if (i_max < 0) return;                               // uniform
    // q rows (scaled) into LDS
    for (int idx = tid; idx < ATT_NQ * DkP; idx += ATT_THREADS) {
        const int r = idx / DkP, d = idx % DkP;
        float v = 0.f;
        if (rpos[r] >= 0 && d < Dk) {
            const int tq = r / HPW, h = g * rep + chunk * HPW + r % HPW;
            v = ldf<T>(q + ((long)b * S + t0 + tq) * qstride + (long)h * Dk + d) * (scale * rtemp[r]);
        }
        qs[idx] = v;
    }
    __syncthreads();

    const int* bt = btab + (long)b * max_blocks;
    const int lo = max(max(0, i_min - window + 1), cmask > 0 ? (i_min / cmask) * cmask : 0);
    const int nfirst = min(keep, lo);
    const int n = nfirst + (i_max - lo + 1);
    const int ntiles = (n + WAVE - 1) / WAVE;
    const int rounds = (ntiles + ATT_WAVES - 1) / ATT_WAVES;
    float m_run[ATT_NQ], l_run[ATT_NQ], acc[ATT_NQ][MAXR];
#pragma unroll
    for (int r = 0; r < ATT_NQ; ++r) {
        m_run[r] = -INFINITY; l_run[r] = 0.f;
#pragma unroll
        for (int c = 0; c < MAXR; ++c) acc[r][c] = 0.f;
    }
    float* myp = ps + wv * pws;
    constexpr int NV = ATT_NQ == 4 ? 8 : 1;
    float acc8[ATT_NQ == 4 ? 4 : 1][NV];
#pragma unroll
    for (int r = 0; r < (ATT_NQ == 4 ? 4 : 1); ++r)
#pragma unroll
        for (int e = 0; e < NV; ++e) acc8[r][e] = 0.f;

    for (int rd = 0; rd < rounds; ++rd) {
        const int base = (rd * ATT_WAVES + wv) * WAVE;
        const int m = base + lane;
        const bool kvalid = m < n;
        int j = 0;
        long slot = 0;
        float sc[ATT_NQ];
#pragma unroll
        for (int r = 0; r < ATT_NQ; ++r) sc[r] = 0.f;
        if (base < n) {                                  // wave-uniform
            if (kvalid) {
                j = m < nfirst ? m : lo + (m - nfirst);
                const int blk = bt[j / bsz];
                slot = (long)(blk < 0 ? 0 : blk) * bsz + (j % bsz);
            }
            const T* kp = kc + slot * ktok + (long)g * khead;
            if (kvec) {
                for (int d = 0; d < Dk; d += 8) {
                    float kv[8];
                    load8<T>(kp + d, kv);
#pragma unroll
                    for (int r = 0; r < ATT_NQ; ++r) {
                        if (rpos[r] < 0) continue;       // uniform
                        const float4 qa = *reinterpret_cast<const float4*>(qs + r * DkP + d);
                        const float4 qb = *reinterpret_cast<const float4*>(qs + r * DkP + d + 4);
                        sc[r] += kv[0] * qa.x + kv[1] * qa.y + kv[2] * qa.z + kv[3] * qa.w +
                                 kv[4] * qb.x + kv[5] * qb.y + kv[6] * qb.z + kv[7] * qb.w;
                    }
                }
            } else {
                for (int d = 0; d < Dk; ++d) {
                    const float kvs = ldf<T>(kp + d);
#pragma unroll
                    for (int r = 0; r < ATT_NQ; ++r) sc[r] += kvs * qs[r * DkP + d];
                }
            }
            // bias, mask, online softmax per row
#pragma unroll
            for (int r = 0; r < ATT_NQ; ++r) {
                const int i = rpos[r];
                if (i < 0) continue;                     // uniform
                const int dist = i - j;
                const bool vis = kvalid && dist >= 0 && (dist < window || j < keep) &&
                                 j >= rclo[r];
                float sv = -INFINITY;
                if (vis) {
                    sv = sc[r];
                    if (r1 && r2) {                      // uniform
                        const float x = ra2[r] * (float)dist;
                        const float lg = sizeof(T) == 4 ? log1pf(x) : __logf(1.f + x);
                        sv -= ra1[r] * lg;
                    } else if (r1) {
                        sv -= ra1[r] * (float)dist;
                    }
                    if (cap > 0.f) sv = cap * tanhf(sv / cap);
                }
                const float m_new = fmaxf(m_run[r], wave_max(sv));
                float p = 0.f, corr = 1.f;
                if (m_new > -INFINITY) {
                    p = vis ? expf(sv - m_new) : 0.f;
                    corr = expf(m_run[r] - m_new);
                }
                l_run[r] = l_run[r] * corr + wave_sum(p);
                m_run[r] = m_new;
#pragma unroll
                for (int c = 0; c < MAXR; ++c) acc[r][c] *= corr;
                if constexpr (ATT_NQ == 4) {
#pragma unroll
                    for (int e = 0; e < NV; ++e) acc8[r][e] *= corr;
                }
                sc[r] = p;
            }
#pragma unroll
            for (int r = 0; r < ATT_NQ; ++r) myp[lane * ATT_NQ + r] = sc[r];
        }
        __syncthreads();
        if (base < n) {
            const int cnt = min(WAVE, n - base);
            const int sl = (int)slot;
            bool done = false;
            if constexpr (ATT_NQ == 4) {
                if (lpr > 0) {
                    done = true;
                    const int ksub = WAVE / lpr;
                    const int sub = lane / lpr, ch = (lane % lpr) * 8;
                    for (int it = 0; it * ksub < cnt; ++it) {
                        const int mm = it * ksub + sub;
                        const long sj = __shfl(sl, mm < cnt ? mm : 0, WAVE);
                        if (mm < cnt) {
                            float vv[8];
                            load8<T>(vc + sj * vtok + (long)g * vhead + ch, vv);
                            const float4 pp = *reinterpret_cast<const float4*>(myp + mm * ATT_NQ);
#pragma unroll
                            for (int e = 0; e < 8; ++e) {
                                acc8[0][e] += pp.x * vv[e];
                                acc8[1][e] += pp.y * vv[e];
                                acc8[2][e] += pp.z * vv[e];
                                acc8[3][e] += pp.w * vv[e];
                            }
                        }
                    }
                }
            }
            if (!done) {
                for (int mm = 0; mm < cnt; ++mm) {
                    const long sj = __shfl(sl, mm, WAVE);
                    const T* vp = vc + sj * vtok + (long)g * vhead;
                    float vv[MAXR];
#pragma unroll
                    for (int c = 0; c < MAXR; ++c) {
                        const int d = lane + c * WAVE;
                        vv[c] = d < Dv ? ldf<T>(vp + d) : 0.f;
                    }
                    const float4* p4 = reinterpret_cast<const float4*>(myp + mm * ATT_NQ);
#pragma unroll
                    for (int r4 = 0; r4 < ATT_NQ / 4; ++r4) {
                        const float4 pp = p4[r4];
#pragma unroll
                        for (int c = 0; c < MAXR; ++c) {
                            acc[4 * r4][c] += pp.x * vv[c];
                            acc[4 * r4 + 1][c] += pp.y * vv[c];
                            acc[4 * r4 + 2][c] += pp.z * vv[c];
                            acc[4 * r4 + 3][c] += pp.w * vv[c];
                        }
                    }
                }
            }
        }
        __syncthreads();
    }
    if constexpr (ATT_NQ == 4) {
        if (lpr > 0) {
            // fold the key subgroups, then move to the channel-per-lane layout
            // the merge and the epilogue use (through this wave's LDS region)
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float v = acc8[r][e];
                    for (int off = lpr; off < WAVE; off <<= 1) v += __shfl_xor(v, off, WAVE);
                    if (lane < lpr) myp[r * Dv + lane * 8 + e] = v;
                }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < MAXR; ++c) {
                    const int d = lane + c * WAVE;
                    if (d < Dv) acc[r][c] = myp[r * Dv + d];
                }
            __syncthreads();
        }
    }
    // merge the waves' partial softmaxes pairwise (tree) through LDS
    for (int step = 1; step < ATT_WAVES; step <<= 1) {
        float* slot_acc = cs + (wv / (2 * step)) * ATT_NQ * (Dv + 2);
        float* cm = slot_acc + ATT_NQ * Dv;
        float* cl = cm + ATT_NQ;
        if (wv % (2 * step) == step) {
#pragma unroll
            for (int r = 0; r < ATT_NQ; ++r) {
                if (lane == 0) { cm[r] = m_run[r]; cl[r] = l_run[r]; }
#pragma unroll
                for (int c = 0; c < MAXR; ++c) {
                    const int d = lane + c * WAVE;
                    if (d < Dv) slot_acc[r * Dv + d] = acc[r][c];
                }
            }
        }
        __syncthreads();
        if (wv % (2 * step) == 0 && wv + step < ATT_WAVES) {
#pragma unroll
            for (int r = 0; r < ATT_NQ; ++r) {
                const float mo = cm[r], lo2 = cl[r];
                const float m_new = fmaxf(m_run[r], mo);
                float ca = 1.f, cb = 0.f;
                if (m_new > -INFINITY) { ca = expf(m_run[r] - m_new); cb = expf(mo - m_new); }
                l_run[r] = l_run[r] * ca + lo2 * cb;
                m_run[r] = m_new;
#pragma unroll
                for (int c = 0; c < MAXR; ++c) {
                    const int d = lane + c * WAVE;
                    if (d < Dv) acc[r][c] = acc[r][c] * ca + slot_acc[r * Dv + d] * cb;
                }
            }
        }
        __syncthreads();
    }
    if (wv != 0) return;
#pragma unroll
    for (int r = 0; r < ATT_NQ; ++r) {
        if (rpos[r] < 0) continue;
        const int tq = r / HPW, h = g * rep + chunk * HPW + r % HPW;
        const long tok = (long)b * S + t0 + tq;
        float inv = 1.f / l_run[r];
        if (sink) {                                      // one more term in the denominator
            const float mf = fmaxf(m_run[r], rsink[r]);
            const float ca = expf(m_run[r] - mf);
            inv = ca / (l_run[r] * ca + expf(rsink[r] - mf));
        }
        TOut* op = out + (tok * H + h) * (long)Dv;
        // gate: one number per value channel, or (ghead) one per head
        const T* gp = gate ? gate + tok * gstride + (ghead ? (long)h : (long)h * Dv) : nullptr;
        if (gp && ghead) inv *= sigmoidf_(ldf<T>(gp));
        if (ghead) gp = nullptr;
#pragma unroll
        for (int c = 0; c < MAXR; ++c) {
            const int d = lane + c * WAVE;
            if (d < Dv) {
                float o = acc[r][c] * inv;
                if (gp) o *= sigmoidf_(ldf<T>(gp + d));
                stf<TOut>(op + d, o);
            }
        }
    }
}

// -------------------------------------------------- paged attention, matrix cores
// bf16 prompt-portion path, same scores and options as above. Workgroup = 64
// query rows of one KV head (4 waves x 16 rows: the group's heads x consecutive
// tokens); all waves walk the same 64-key tiles, staged once in LDS (K row-major,
// V transposed). Scores are computed transposed, S^T = K Q^T (mfma 16x16x32 bf16,
// fp32 accumulate), so a lane ends up with 16 scores of ONE query row and the
// probabilities already sit in the A-operand layout of the P.V product. Scale,
// temperature, bias, cap, mask and online softmax are fp32 per lane; P enters the
// second product as a hi + lo bf16 pair (16 mantissa bits), V as stored.
// DKP / DVP are the head sizes padded to multiples of 32; the true Dk, Dv (any
// multiples of 8) come at run time and the padding is zero-filled in LDS. KT is
// the key tile (64, or 32 for wide keys so that the K tile still fits LDS). Values
// wider than DVP are split over `nsplit` workgroups that each recompute the scores
// and own DVP value channels (latent caches: a 576-wide key row whose first 512
// channels are the value).
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
#define MA_ROWS 64

DEV uint16_t f2bf_rne(float f) {
    uint32_t u = __float_as_uint(f);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// bf16-only kernels take the hardware exponential: its 2^-21 relative error is
// far below the rounding of their operands
DEV float fast_tanh_(float y) { return 1.f - __fdividef(2.f, 1.f + __expf(2.f * y)); }

template <int DKP, int DVP, int MA_KT, bool PREFETCH>
__global__ void __launch_bounds__(256)
paged_attn_mfma_kernel(const bf16* __restrict__ q, long qstride, const bf16* __restrict__ kc,
                       const bf16* __restrict__ vc, const int* __restrict__ pos,
                       const int* __restrict__ seq, const int* __restrict__ btab,
                       int max_blocks, const float* __restrict__ r1,
                       const float* __restrict__ r2, const bf16* __restrict__ gate,
                       long gstride, bf16* __restrict__ out, int H, int G, int Dk, int Dv,
                       int bsz, int S, float scale, int window, int keep, int QT, long ktok,
                       long khead, long vtok, long vhead, const float* __restrict__ sink,
                       float cap, float qt_coef, int qt_every, int nsplit, int ghead,
                       int cmask) {
    constexpr int KB = MA_KT / 16;           // 16-key score blocks per tile
    constexpr int KS = DKP + 8;              // K tile row stride (elements)
    constexpr int VS = MA_KT + 8;            // V^T tile row stride
    __shared__ __attribute__((aligned(16))) uint16_t k_lds[MA_KT * KS];
    __shared__ __attribute__((aligned(16))) uint16_t vt_lds[DVP * VS];
    __shared__ int rpos[MA_ROWS];
    __shared__ float ra1[MA_ROWS], ra2[MA_ROWS], rsink[MA_ROWS];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int lr = lane & 15, lg = lane >> 4;
    const int b = blockIdx.z, g = blockIdx.y / nsplit, t0 = blockIdx.x * QT;
    const int dv0 = (blockIdx.y % nsplit) * DVP;         // first value channel of this split
    const int dvn = min(DVP, Dv - dv0);
    const int rep = H / G;
    if (seq[b] < 0) return;
    if (tid < MA_ROWS) {
        const int tq = tid / rep, hh = tid % rep;
        rpos[tid] = (tq < QT && t0 + tq < S) ? pos[(long)b * S + t0 + tq] : -1;
        ra1[tid] = r1 ? r1[g * rep + hh] : 0.f;
        ra2[tid] = r2 ? r2[g * rep + hh] : 0.f;
        rsink[tid] = sink ? sink[g * rep + hh] : -INFINITY;
    }
    __syncthreads();
    int i_min = 0x7fffffff, i_max = -1;
    for (int r = 0; r < MA_ROWS; r += rep) {     // one entry per token
        const int p = rpos[r];
        if (p >= 0) { i_min = min(i_min, p); i_max = max(i_max, p); }
    }
    if (i_max < 0) return;                       // uniform
    // this lane's query row (B operand of S^T): row = 16*wv + lr
    const int myrow = wv * 16 + lr;
    const int my_i = rpos[myrow];
    const int my_clo = (cmask > 0 && my_i >= 0) ? (my_i / cmask) * cmask : 0;
    const float a1 = ra1[myrow], a2 = ra2[myrow];
    const float qscale = (qt_every > 0 && my_i >= 0)
        ? scale * (1.f + qt_coef * logf((float)((my_i + 1) / qt_every) + 1.f)) : scale;
    bf16x8_t qf[DKP / 32];
    {
        const int tq = myrow / rep, h = g * rep + myrow % rep;
        const bf16* qp = q + ((long)b * S + t0 + tq) * qstride + (long)h * Dk;
#pragma unroll
        for (int ks = 0; ks < DKP / 32; ++ks) {
            uint4 raw = make_uint4(0, 0, 0, 0);
            if (my_i >= 0 && ks * 32 + lg * 8 < Dk)
                raw = *reinterpret_cast<const uint4*>(qp + ks * 32 + lg * 8);
            qf[ks] = *reinterpret_cast<bf16x8_t*>(&raw);
        }
    }
    const int* bt = btab + (long)b * max_blocks;
    const int lo = max(max(0, i_min - window + 1), cmask > 0 ? (i_min / cmask) * cmask : 0);
    const int clo_max = cmask > 0 ? (i_max / cmask) * cmask : 0;   // block start of the last row
    const int nfirst = min(keep, lo);
    const int n = nfirst + (i_max - lo + 1);
    float m_run = -INFINITY, l_run = 0.f;
    f32x4_t o_acc[DVP / 16];
#pragma unroll
    for (int nb = 0; nb < DVP / 16; ++nb) o_acc[nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // a tile's K and V lines travel global -> registers -> LDS. With PREFETCH
    // (wide rows: one workgroup per CU, nothing else to hide latency) the next
    // tile's loads are issued before the current tile's products; without, the
    // registers are reused and more workgroups share a CU
    constexpr int NKI = (MA_KT * (DKP / 8) + 255) / 256;
    constexpr int NVI = (MA_KT * (DVP / 8) + 255) / 256;
    uint4 rk[NKI], rv[NVI];
#define MA_FETCH(BASE)                                                                     \
    {                                                                                      \
        _Pragma("unroll") for (int x = 0; x < NKI; ++x) {                                  \
            const int c = tid + x * 256;                                                   \
            const int m = c / (DKP / 8), part = c % (DKP / 8);                             \
            uint4 raw = make_uint4(0, 0, 0, 0);                                            \
            if (c < MA_KT * (DKP / 8) && (BASE) + m < n && part * 8 < Dk) {                \
                const int mm = (BASE) + m;                                                 \
                const int j = mm < nfirst ? mm : lo + (mm - nfirst);                       \
                const int blk = bt[j / bsz];                                               \
                const long slot = (long)(blk < 0 ? 0 : blk) * bsz + (j % bsz);             \
                raw = *reinterpret_cast<const uint4*>(kc + slot * ktok + (long)g * khead + part * 8); \
            }                                                                              \
            rk[x] = raw;                                                                   \
        }                                                                                  \
        _Pragma("unroll") for (int x = 0; x < NVI; ++x) {                                  \
            const int c = tid + x * 256;                                                   \
            const int m = c % MA_KT, part = c / MA_KT;   /* consecutive lanes: consecutive keys */ \
            uint4 raw = make_uint4(0, 0, 0, 0);                                            \
            if (c < MA_KT * (DVP / 8) && (BASE) + m < n && part * 8 < dvn) {               \
                const int mm = (BASE) + m;                                                 \
                const int j = mm < nfirst ? mm : lo + (mm - nfirst);                       \
                const int blk = bt[j / bsz];                                               \
                const long slot = (long)(blk < 0 ? 0 : blk) * bsz + (j % bsz);             \
                raw = *reinterpret_cast<const uint4*>(vc + slot * vtok + (long)g * vhead + dv0 + \
                                                      part * 8);                           \
            }                                                                              \
            rv[x] = raw;                                                                   \
        }                                                                                  \
    }
    if constexpr (PREFETCH) MA_FETCH(0)
    for (int base = 0; base < n; base += MA_KT) {
        if constexpr (!PREFETCH) {
            // ---- global -> LDS directly: K row-major, V transposed
            for (int c = tid; c < MA_KT * (DKP / 8); c += 256) {
                const int m = c / (DKP / 8), part = c % (DKP / 8);
                uint4 raw = make_uint4(0, 0, 0, 0);
                if (base + m < n && part * 8 < Dk) {
                    const int mm = base + m;
                    const int j = mm < nfirst ? mm : lo + (mm - nfirst);
                    const int blk = bt[j / bsz];
                    const long slot = (long)(blk < 0 ? 0 : blk) * bsz + (j % bsz);
                    raw = *reinterpret_cast<const uint4*>(kc + slot * ktok + (long)g * khead + part * 8);
                }
                *reinterpret_cast<uint4*>(k_lds + m * KS + part * 8) = raw;
            }
            for (int c = tid; c < MA_KT * (DVP / 8); c += 256) {
                const int m = c % MA_KT, part = c / MA_KT;   // consecutive lanes: consecutive keys
                uint4 raw = make_uint4(0, 0, 0, 0);
                if (base + m < n && part * 8 < dvn) {
                    const int mm = base + m;
                    const int j = mm < nfirst ? mm : lo + (mm - nfirst);
                    const int blk = bt[j / bsz];
                    const long slot = (long)(blk < 0 ? 0 : blk) * bsz + (j % bsz);
                    raw = *reinterpret_cast<const uint4*>(vc + slot * vtok + (long)g * vhead + dv0 +
                                                          part * 8);
                }
                const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    vt_lds[(part * 8 + 2 * e) * VS + m] = (uint16_t)(u[e] & 0xffffu);
                    vt_lds[(part * 8 + 2 * e + 1) * VS + m] = (uint16_t)(u[e] >> 16);
                }
            }
        }
        // ---- (prefetched) registers -> LDS
        if constexpr (PREFETCH) {
#pragma unroll
        for (int x = 0; x < NKI; ++x) {
            const int c = tid + x * 256;
            if (c < MA_KT * (DKP / 8))
                *reinterpret_cast<uint4*>(k_lds + (c / (DKP / 8)) * KS + (c % (DKP / 8)) * 8) = rk[x];
        }
#pragma unroll
        for (int x = 0; x < NVI; ++x) {
            const int c = tid + x * 256;
            if (c < MA_KT * (DVP / 8)) {
                const int m = c % MA_KT, part = c / MA_KT;
                const uint32_t u[4] = {rv[x].x, rv[x].y, rv[x].z, rv[x].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    vt_lds[(part * 8 + 2 * e) * VS + m] = (uint16_t)(u[e] & 0xffffu);
                    vt_lds[(part * 8 + 2 * e + 1) * VS + m] = (uint16_t)(u[e] >> 16);
                }
            }
        }
        }
        __syncthreads();
        if constexpr (PREFETCH) {
            if (base + MA_KT < n) MA_FETCH(base + MA_KT) // in flight during the products below
        }
        // ---- S^T = K Q^T: lane gets keys 16*kb + 4*lg + r of its own row lr
        float sv[KB][4];
        float mt = -INFINITY;
        // a tile every row of the workgroup sees whole (all but the diagonal
        // tiles of a causal prompt) needs no per-score mask
        const bool whole = nfirst == 0 && base + MA_KT <= n && lo + base + MA_KT - 1 <= i_min &&
                           i_max - (lo + base) < window && lo + base >= clo_max;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < DKP / 32; ++ks) {
                const bf16x8_t ka = *reinterpret_cast<const bf16x8_t*>(
                    k_lds + (kb * 16 + lr) * KS + ks * 32 + lg * 8);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qf[ks], acc, 0, 0, 0);
            }
            if (whole && !r2) {                          // uniform
                // (a linear penalty needs no mask either: the tile's keys are
                // lo + base + 16 kb + 4 lg + r, all at or before every row)
                const float d0 = (float)(my_i - (lo + base + kb * 16 + lg * 4));
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float x = acc[r] * qscale;
                    if (r1) x -= a1 * (d0 - (float)r);
                    if (cap > 0.f) x = cap * fast_tanh_(x / cap);
                    if (my_i < 0) x = -INFINITY;
                    sv[kb][r] = x;
                    mt = fmaxf(mt, x);
                }
                continue;
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int mm = base + kb * 16 + lg * 4 + r;
                const int j = mm < nfirst ? mm : lo + (mm - nfirst);
                const int dist = my_i - j;
                const bool vis = mm < n && my_i >= 0 && dist >= 0 && (dist < window || j < keep) &&
                                 j >= my_clo;
                float x = -INFINITY;
                if (vis) {
                    x = acc[r] * qscale;
                    if (r1) x -= r2 ? a1 * __logf(1.f + a2 * (float)dist) : a1 * (float)dist;
                    if (cap > 0.f) x = cap * fast_tanh_(x / cap);
                }
                sv[kb][r] = x;
                mt = fmaxf(mt, x);
            }
        }
        mt = fmaxf(mt, __shfl_xor(mt, 16, WAVE));
        mt = fmaxf(mt, __shfl_xor(mt, 32, WAVE));
        const float m_new = fmaxf(m_run, mt);
        float corr = 1.f, psum = 0.f;
        if (m_new > -INFINITY) {
            corr = __expf(m_run - m_new);
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float pv = sv[kb][r] > -INFINITY ? __expf(sv[kb][r] - m_new) : 0.f;
                    sv[kb][r] = pv;
                    psum += pv;
                }
        } else {
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int r = 0; r < 4; ++r) sv[kb][r] = 0.f;
        }
        psum += __shfl_xor(psum, 16, WAVE);
        psum += __shfl_xor(psum, 32, WAVE);
        l_run = l_run * corr + psum;
        m_run = m_new;
        // ---- rescale O: its rows are 4*lg + r, their corr sits in lane (4*lg + r)
        if (__any(corr != 1.f)) {                        // some row's maximum moved
            float cr[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) cr[r] = __shfl(corr, lg * 4 + r, WAVE);
#pragma unroll
            for (int nb = 0; nb < DVP / 16; ++nb)
#pragma unroll
                for (int r = 0; r < 4; ++r) o_acc[nb][r] *= cr[r];
        }
        // ---- O += P V, 32 keys per product, P as hi + lo
#pragma unroll
        for (int kc2 = 0; kc2 < MA_KT / 32; ++kc2) {
            struct { bf16x8_t v; } ph, pl;               // hardware float -> bf16 (RNE)
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) {
                const float pv = sv[2 * kc2 + (jj >> 2)][jj & 3];
                const __bf16 hb = (__bf16)pv;
                ph.v[jj] = hb;
                pl.v[jj] = (__bf16)(pv - (float)hb);
            }
#pragma unroll
            for (int nb = 0; nb < DVP / 16; ++nb) {
                union { bf16x8_t v; uint2 h[2]; } vb;
                const uint16_t* vp = vt_lds + (nb * 16 + lr) * VS + 32 * kc2 + 4 * lg;
                vb.h[0] = *reinterpret_cast<const uint2*>(vp);
                vb.h[1] = *reinterpret_cast<const uint2*>(vp + 16);
                o_acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ph.v, vb.v, o_acc[nb], 0, 0, 0);
                o_acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pl.v, vb.v, o_acc[nb], 0, 0, 0);
            }
        }
        __syncthreads();
    }
#undef MA_FETCH
    // ---- epilogue: rows 4*lg + r of this wave, channel 16*nb + lr. A sink adds
    // one term to the row's denominator (computed by the lane that owns the row)
    float fin = l_run > 0.f ? 1.f / l_run : 0.f;
    if (sink) {
        const float sk = rsink[myrow];
        const float mf = fmaxf(m_run, sk);
        const float ca = m_run > -INFINITY ? __expf(m_run - mf) : 0.f;
        fin = ca / (l_run * ca + __expf(sk - mf));
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = wv * 16 + lg * 4 + r;
        const float inv = __shfl(fin, lg * 4 + r, WAVE);
        if (rpos[row] < 0) continue;
        const int tq = row / rep, h = g * rep + row % rep;
        const long tok = (long)b * S + t0 + tq;
        bf16* op = out + (tok * H + h) * (long)Dv + dv0;
        const bf16* gp = (gate && !ghead) ? gate + tok * gstride + (long)h * Dv + dv0 : nullptr;
        const float hg = (gate && ghead)
            ? sigmoidf_(__bfloat162float(gate[tok * gstride + h])) : 1.f;
#pragma unroll
        for (int nb = 0; nb < DVP / 16; ++nb) {
            const int d = nb * 16 + lr;
            if (d >= dvn) continue;
            float o = o_acc[nb][r] * inv * hg;
            if (gp) o *= sigmoidf_(__bfloat162float(gp[d]));
            op[d] = __float2bfloat16(o);
        }
    }
}

// ------------------------------------ latent-cache decode, matrix cores
// Single-token steps of multi-query layers whose values are the first Dv
// channels of the (one) key row per token — the absorbed form of latent
// attention: 16 query heads of one token are the 16 rows of the score tile.
// All four waves compute the (cheap) scores of a 32-key tile; wave w owns value
// channels [128w, 128w+128), so a workgroup covers 512 of them and the key row
// is fetched from memory once: global -> registers (next tile prefetched) -> LDS
// row-major, then V^T is cut out of that LDS tile. Causal, optionally inside a
// sliding window or the token's block of positions; optional sink.
// Grid: (tokens x key splits, head chunks of 16 x value splits of 512, batch
// rows). With nks > 1 key splits a workgroup scans every nks-th run of tiles and
// leaves an unnormalised partial (fp32 values, running max, sum) in `ws`;
// latent_decode_merge_kernel folds the splits and the sink.
#define LD_KT 32
#define LD_VW 128                            // value channels per wave

template <int DKP>
__global__ void __launch_bounds__(256)
latent_decode_mfma_kernel(const bf16* __restrict__ q, long qstride, const bf16* __restrict__ kc,
                          long ktok, const int* __restrict__ pos, const int* __restrict__ seq,
                          const int* __restrict__ btab, int max_blocks,
                          const float* __restrict__ sink, bf16* __restrict__ out, int H, int Dk,
                          int Dv, int bsz, int S, float scale, int nsplit, int nks,
                          float* __restrict__ ws, int window, int cmask) {
    constexpr int KS = DKP + 8;
    constexpr int VS = LD_KT + 8;
    constexpr int VCH = 4 * LD_VW;
    extern __shared__ __attribute__((aligned(16))) uint16_t ld_lds[];
    uint16_t* k_lds = ld_lds;                            // LD_KT * KS
    uint16_t* vt_lds = ld_lds + LD_KT * KS;              // VCH * VS
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int lr = lane & 15, lg = lane >> 4;
    const int b = blockIdx.z, t = blockIdx.x / nks, ksp = blockIdx.x % nks;
    const int h0 = (blockIdx.y / nsplit) * 16;
    const int dv0 = (blockIdx.y % nsplit) * VCH;         // this workgroup's first value channel
    const int dvn = min(VCH, Dv - dv0);
    if (seq[b] < 0) return;
    const int p = pos[(long)b * S + t];
    if (p < 0) return;                                   // uniform
    const int h = h0 + lr;                               // this lane's query row
    const bool hv = h < H;
    bf16x8_t qf[DKP / 32];
    {
        const bf16* qp = q + ((long)b * S + t) * qstride + (long)h * Dk;
#pragma unroll
        for (int ks = 0; ks < DKP / 32; ++ks) {
            uint4 raw = make_uint4(0, 0, 0, 0);
            if (hv && ks * 32 + lg * 8 < Dk) raw = *reinterpret_cast<const uint4*>(qp + ks * 32 + lg * 8);
            qf[ks] = *reinterpret_cast<bf16x8_t*>(&raw);
        }
    }
    const int* bt = btab + (long)b * max_blocks;
    // the token sees keys [first, p]; this split's keys [k_lo, n) are a
    // contiguous run of 32-key tiles counted from `first`
    const int first = max(max(0, p - window + 1), cmask > 0 ? (p / cmask) * cmask : 0);
    const int tiles = (p + 1 - first + LD_KT - 1) / LD_KT, per = (tiles + nks - 1) / nks;
    const int k_lo = first + ksp * per * LD_KT;
    const int n = min(p + 1, first + (ksp + 1) * per * LD_KT);
    float m_run = -INFINITY, l_run = 0.f;
    f32x4_t o_acc[LD_VW / 16];
#pragma unroll
    for (int nb = 0; nb < LD_VW / 16; ++nb) o_acc[nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    constexpr int NKI = (LD_KT * (DKP / 8) + 255) / 256;
    uint4 rk[NKI];
#define LD_FETCH(BASE)                                                                     \
    _Pragma("unroll") for (int x = 0; x < NKI; ++x) {                                      \
        const int c = tid + x * 256;                                                       \
        const int m = c / (DKP / 8), part = c % (DKP / 8);                                 \
        uint4 raw = make_uint4(0, 0, 0, 0);                                                \
        if (c < LD_KT * (DKP / 8) && (BASE) + m < n && part * 8 < Dk) {                    \
            const int j = (BASE) + m;                                                      \
            const int blk = bt[j / bsz];                                                   \
            const long slot = (long)(blk < 0 ? 0 : blk) * bsz + (j % bsz);                 \
            raw = *reinterpret_cast<const uint4*>(kc + slot * ktok + part * 8);            \
        }                                                                                  \
        rk[x] = raw;                                                                       \
    }
    LD_FETCH(k_lo)
    for (int base = k_lo; base < n; base += LD_KT) {
#pragma unroll
        for (int x = 0; x < NKI; ++x) {
            const int c = tid + x * 256;
            if (c < LD_KT * (DKP / 8))
                *reinterpret_cast<uint4*>(k_lds + (c / (DKP / 8)) * KS + (c % (DKP / 8)) * 8) = rk[x];
        }
        __syncthreads();
        if (base + LD_KT < n) LD_FETCH(base + LD_KT)     // in flight during the work below
        // ---- V^T (channels dv0..dv0+dvn) out of the K tile
        for (int c = tid; c < LD_KT * (VCH / 8); c += 256) {
            const int m = c % LD_KT, part = c / LD_KT;
            uint4 raw = make_uint4(0, 0, 0, 0);
            if (part * 8 < dvn) raw = *reinterpret_cast<const uint4*>(k_lds + m * KS + dv0 + part * 8);
            const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                vt_lds[(part * 8 + 2 * e) * VS + m] = (uint16_t)(u[e] & 0xffffu);
                vt_lds[(part * 8 + 2 * e + 1) * VS + m] = (uint16_t)(u[e] >> 16);
            }
        }
        // ---- S^T = K Q^T: lane gets keys 16*kb + 4*lg + r of row lr
        float sv[2][4];
        float mt = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < DKP / 32; ++ks) {
                const bf16x8_t ka = *reinterpret_cast<const bf16x8_t*>(
                    k_lds + (kb * 16 + lr) * KS + ks * 32 + lg * 8);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qf[ks], acc, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int j = base + kb * 16 + lg * 4 + r;
                const float x = (j < n && hv) ? acc[r] * scale : -INFINITY;
                sv[kb][r] = x;
                mt = fmaxf(mt, x);
            }
        }
        mt = fmaxf(mt, __shfl_xor(mt, 16, WAVE));
        mt = fmaxf(mt, __shfl_xor(mt, 32, WAVE));
        const float m_new = fmaxf(m_run, mt);
        float corr = 1.f, psum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float pv = (m_new > -INFINITY && sv[kb][r] > -INFINITY)
                    ? __expf(sv[kb][r] - m_new) : 0.f;
                sv[kb][r] = pv;
                psum += pv;
            }
        if (m_new > -INFINITY) corr = __expf(m_run - m_new);
        psum += __shfl_xor(psum, 16, WAVE);
        psum += __shfl_xor(psum, 32, WAVE);
        l_run = l_run * corr + psum;
        m_run = m_new;
        float cr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) cr[r] = __shfl(corr, lg * 4 + r, WAVE);
#pragma unroll
        for (int nb = 0; nb < LD_VW / 16; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) o_acc[nb][r] *= cr[r];
        __syncthreads();                                 // V^T complete
        // ---- O += P V for this wave's 128 channels, P as hi + lo
        {
            struct { bf16x8_t v; } ph, pl;
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) {
                const float pv = sv[jj >> 2][jj & 3];
                const __bf16 hb = (__bf16)pv;
                ph.v[jj] = hb;
                pl.v[jj] = (__bf16)(pv - (float)hb);
            }
#pragma unroll
            for (int nb = 0; nb < LD_VW / 16; ++nb) {
                union { bf16x8_t v; uint2 h2[2]; } vb;
                const uint16_t* vp = vt_lds + (wv * LD_VW + nb * 16 + lr) * VS + 4 * lg;
                vb.h2[0] = *reinterpret_cast<const uint2*>(vp);
                vb.h2[1] = *reinterpret_cast<const uint2*>(vp + 16);
                o_acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ph.v, vb.v, o_acc[nb], 0, 0, 0);
                o_acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pl.v, vb.v, o_acc[nb], 0, 0, 0);
            }
        }
        __syncthreads();
    }
#undef LD_FETCH
    if (nks > 1) {
        // partial result: [(token, head, split)][Dv values | max | sum]
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int hh = h0 + lg * 4 + r;
            const float mr = __shfl(m_run, lg * 4 + r, WAVE), lrn = __shfl(l_run, lg * 4 + r, WAVE);
            if (hh >= H) continue;
            float* wp = ws + ((((long)b * S + t) * H + hh) * nks + ksp) * (long)(Dv + 2);
#pragma unroll
            for (int nb = 0; nb < LD_VW / 16; ++nb) {
                const int d = wv * LD_VW + nb * 16 + lr;
                if (d < dvn) wp[dv0 + d] = o_acc[nb][r];
            }
            if (dv0 == 0 && wv == 0 && lr == 0) { wp[Dv] = mr; wp[Dv + 1] = lrn; }
        }
        return;
    }
    float fin = l_run > 0.f ? 1.f / l_run : 0.f;
    if (sink && hv) {
        const float sk = sink[h];
        const float mf = fmaxf(m_run, sk);
        const float ca = m_run > -INFINITY ? __expf(m_run - mf) : 0.f;
        fin = ca / (l_run * ca + __expf(sk - mf));
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int hh = h0 + lg * 4 + r;
        const float inv = __shfl(fin, lg * 4 + r, WAVE);
        if (hh >= H) continue;
        bf16* op = out + (((long)b * S + t) * H + hh) * (long)Dv + dv0 + wv * LD_VW;
#pragma unroll
        for (int nb = 0; nb < LD_VW / 16; ++nb) {
            const int d = wv * LD_VW + nb * 16 + lr;
            if (d < dvn) op[nb * 16 + lr] = __float2bfloat16(o_acc[nb][r] * inv);
        }
    }
}

// one wave per (token, head): out = sum_i o_i e^(m_i - M) / (sum_i l_i e^(m_i - M)
// + e^(sink - M)), M the largest of the splits' maxima and the sink
__global__ void latent_decode_merge_kernel(const float* __restrict__ ws,
                                           const float* __restrict__ sink,
                                           const int* __restrict__ pos, const int* __restrict__ seq,
                                           bf16* __restrict__ out, long ntok, int S, int H, int Dv,
                                           int nks) {
    const int lane = threadIdx.x & (WAVE - 1);
    const long wid = (long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (wid >= ntok * H) return;
    const long tok = wid / H;
    const int h = wid % H;
    if (pos[tok] < 0 || seq[tok / S] < 0) return;
    const float* wp = ws + wid * nks * (long)(Dv + 2);
    const float sk = sink ? sink[h] : -INFINITY;
    float M = sk;
    for (int i = 0; i < nks; ++i) M = fmaxf(M, wp[i * (long)(Dv + 2) + Dv]);
    float L = sink ? expf(sk - M) : 0.f;
    for (int i = 0; i < nks; ++i) {
        const float mi = wp[i * (long)(Dv + 2) + Dv];
        if (mi > -INFINITY) L += wp[i * (long)(Dv + 2) + Dv + 1] * expf(mi - M);
    }
    const float inv = L > 0.f ? 1.f / L : 0.f;
    float wgt[8];                                        // nks <= 8
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float mi = i < nks ? wp[i * (long)(Dv + 2) + Dv] : -INFINITY;
        wgt[i] = mi > -INFINITY ? expf(mi - M) * inv : 0.f;
    }
    for (int d = lane; d < Dv; d += WAVE) {
        float o = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (i < nks) o += wp[i * (long)(Dv + 2) + d] * wgt[i];
        out[wid * Dv + d] = __float2bfloat16(o);
    }
}

// ------------------------------------------------------- gated delta rule
// Three kernels per step.
// (1) delta_prep_kernel, fully parallel over tokens: unit q and k per KV head
//     (q also scaled by D^-1/2), decay exp(-exp(A_log) softplus(a + dt_bias))
//     per head and key channel, beta = sigmoid(.), all fp32, into one row per
//     token: [q (G*D) | k (G*D) | decay (H*D) | beta (H)], stride PS.
// (2) gated_delta_kernel, the serial scan. Workgroup = (row, head, block of
//     value channels), 256 threads. The (D x Dv) state is kept in registers:
//     16 (8 for D <= 32) adjacent lanes share one value channel (column) and
//     split its D rows in float4-interleaved order, so a token costs D/16
//     multiply-adds per lane plus two DPP lane reductions and no
//     workgroup-wide traffic. Tokens go in chunks of TC through LDS; the next
//     chunk's rows are fetched into registers while the current one is
//     scanned. State memory layout is (slot, head, Dv, D): a lane's rows are
//     contiguous float4s, a column's rows one contiguous line.
// (3) gated_rmsnorm_kernel: per-head RMS norm, weight and sigmoid gate (needs
//     all value channels of a head, which (2) spreads over workgroups).
#define GD_THREADS 256

template <typename T>
__global__ void delta_prep_kernel(const float* __restrict__ qkv, long cstride,
                                  const T* __restrict__ beta, long bstride,
                                  const T* __restrict__ a, long astride,
                                  const float* __restrict__ dt_bias,
                                  const float* __restrict__ a_log, const int* __restrict__ pos,
                                  const int* __restrict__ seq, float* __restrict__ prep, long PS,
                                  long ntok, int S, int H, int G, int D, int per_head) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int units = 2 * G + H;
    const long wid = (long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (wid >= ntok * units) return;
    const long tok = wid / units;
    const int u = wid % units;
    if (pos[tok] < 0 || seq[tok / S] < 0) return;
    float* pr = prep + tok * PS;
    if (u < 2 * G) {
        const float* src = qkv + tok * cstride + (long)u * D;      // q heads then k heads
        float ss = 0.f;
        for (int i = lane; i < D; i += WAVE) { float x = src[i]; ss += x * x; }
        float inv = 1.f / sqrtf(wave_sum(ss) + 1e-6f);
        if (u < G) inv *= 1.f / sqrtf((float)D);
        for (int i = lane; i < D; i += WAVE) pr[(long)u * D + i] = src[i] * inv;
        if (u < G) {
            // q^ . k^ of this KV head: lets the scan read out before it writes
            const float* ksrc = src + (long)G * D;
            float sk = 0.f, qk = 0.f;
            for (int i = lane; i < D; i += WAVE) { float y = ksrc[i]; sk += y * y; qk += src[i] * y; }
            sk = wave_sum(sk);
            qk = wave_sum(qk);
            if (lane == 0)
                pr[(long)(2 * G + H) * D + H + u] = qk * inv * (1.f / sqrtf(sk + 1e-6f));
        }
    } else {
        const int h = u - 2 * G;
        const float neg_rate = -expf(a_log[h]);
        if (per_head) {
            // one decay for the whole head, broadcast over its key channels
            const float dec = expf(neg_rate * softplusf_(ldf<T>(a + tok * astride + h) + dt_bias[h]));
            for (int i = lane; i < D; i += WAVE) pr[(long)(2 * G + h) * D + i] = dec;
        } else {
            const T* ap = a + tok * astride + (long)h * D;
            for (int i = lane; i < D; i += WAVE)
                pr[(long)(2 * G + h) * D + i] =
                    expf(neg_rate * softplusf_(ldf<T>(ap + i) + dt_bias[h * D + i]));
        }
        if (lane == 0)
            pr[(long)(2 * G + H) * D + h] = sigmoidf_(ldf<T>(beta + tok * bstride + h));
    }
}

// sum over the 8 or 16 adjacent lanes that share a value channel, on the DPP
// path (quad xor 1, quad xor 2, mirrored half row, mirrored row: after each
// step every lane of a group holds the group's sum, so any lane of the
// sibling group will do)
template <int PARTS>
DEV float part_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
        0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
        0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
        0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));   // row_half_mirror
    if (PARTS == 16)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
            0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));   // row_mirror
    return v;
}

template <int DK, int TC, int GD_PARTS>
__global__ void __launch_bounds__(GD_THREADS)
gated_delta_kernel(const float* __restrict__ qkv, long cstride, const float* __restrict__ prep,
                   long PS, float* __restrict__ state, const int* __restrict__ pos,
                   const int* __restrict__ seq, const int* __restrict__ nvalid,
                   float* __restrict__ obuf, int S, int H, int G, int D, int Dv) {
    constexpr int GD_CW = GD_THREADS / GD_PARTS;   // value channels per workgroup
    constexpr int R = DK / GD_PARTS;         // rows per lane
    constexpr int F = R / 4;                 // float4s per lane
    constexpr int NQKG = 3 * TC * DK;        // LDS floats per chunk: q | k | decay
    constexpr int NE = NQKG + TC * GD_CW + 2 * TC;   // ... | v (TC x GD_CW) | beta | q.k
    constexpr int PER = (NE + GD_THREADS - 1) / GD_THREADS;
    __shared__ __attribute__((aligned(16))) float buf[PER * GD_THREADS];
    const float* qs = buf;
    const float* ks = buf + TC * DK;
    const float* gs = buf + 2 * TC * DK;
    const float* vs = buf + NQKG;
    const float* bs = vs + TC * GD_CW;
    const float* kqs = bs + TC;
    const int h = blockIdx.y, b = blockIdx.z;
    const int slot = seq[b];
    const int n = nvalid[b];
    if (slot < 0 || n <= 0) return;          // uniform over the workgroup
    const int tid = threadIdx.x;
    const int part = tid % GD_PARTS;
    const int cl = tid / GD_PARTS;
    const int col0 = blockIdx.x * GD_CW;
    const int col = col0 + cl;
    const bool act = col < Dv;
    const int g = h / (H / G);
    const int p0 = pos[(long)b * S];
    float* st = state + (((long)slot * H + h) * Dv + (act ? col : 0)) * D;
    float s[R];
#pragma unroll
    for (int f = 0; f < F; ++f)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = (f * GD_PARTS + part) * 4 + e;
            s[f * 4 + e] = (act && row < D && p0 > 0) ? st[row] : 0.f;
        }
    const long off_q = (long)g * D, off_k = (long)(G + g) * D, off_g = (long)(2 * G + h) * D;
    const long off_b = (long)(2 * G + H) * D + h;
    const long off_kq = (long)(2 * G + H) * D + H + g;
    const long off_v = 2L * G * D + (long)h * Dv + col0;

    float pre[PER];
    // chunk at t0 -> registers (loads are issued, not waited for)
#define GD_FETCH(T0)                                                                      \
    {                                                                                     \
        const int ftc = min(TC, n - (T0));                                                \
        const long frow = (long)b * S + (T0);                                             \
        _Pragma("unroll") for (int x = 0; x < PER; ++x) {                                 \
            const int idx = tid + x * GD_THREADS;                                         \
            float v = 0.f;                                                                \
            if (idx < NQKG) {                                                             \
                const int which = idx / (TC * DK), rem = idx % (TC * DK);                 \
                const int tk = rem / DK, i = rem % DK;                                    \
                if (tk < ftc && i < D)                                                    \
                    v = prep[(frow + tk) * PS + (which == 0 ? off_q : which == 1 ? off_k : off_g) + i]; \
            } else if (idx < NQKG + TC * GD_CW) {                                         \
                const int tk = (idx - NQKG) / GD_CW, c = (idx - NQKG) % GD_CW;            \
                if (tk < ftc && col0 + c < Dv) v = qkv[(frow + tk) * cstride + off_v + c]; \
            } else if (idx < NE) {                                                        \
                const int e = idx - NQKG - TC * GD_CW;                                    \
                const int tk = e % TC;                                                    \
                if (tk < ftc) v = prep[(frow + tk) * PS + (e < TC ? off_b : off_kq)];     \
            }                                                                             \
            pre[x] = v;                                                                   \
        }                                                                                 \
    }
    GD_FETCH(0)
    for (int t0 = 0; t0 < n; t0 += TC) {
        const int tc = min(TC, n - t0);
        const long row0 = (long)b * S + t0;
#pragma unroll
        for (int x = 0; x < PER; ++x) buf[tid + x * GD_THREADS] = pre[x];
        __syncthreads();
        if (t0 + TC < n) GD_FETCH(t0 + TC)   // in flight during the scan below
#pragma unroll 2
        for (int tk = 0; tk < tc; ++tk) {
            const float4* g4 = reinterpret_cast<const float4*>(gs + tk * DK) + part;
            const float4* k4 = reinterpret_cast<const float4*>(ks + tk * DK) + part;
            const float4* q4 = reinterpret_cast<const float4*>(qs + tk * DK) + part;
            float4 kk[F];
            float dot = 0.f, oq = 0.f;       // (dS)^T k and (dS)^T q, this lane's rows
#pragma unroll
            for (int f = 0; f < F; ++f) {
                const float4 gg = g4[f * GD_PARTS];
                const float4 qq = q4[f * GD_PARTS];
                kk[f] = k4[f * GD_PARTS];
                s[4 * f] *= gg.x; dot += s[4 * f] * kk[f].x; oq += s[4 * f] * qq.x;
                s[4 * f + 1] *= gg.y; dot += s[4 * f + 1] * kk[f].y; oq += s[4 * f + 1] * qq.y;
                s[4 * f + 2] *= gg.z; dot += s[4 * f + 2] * kk[f].z; oq += s[4 * f + 2] * qq.z;
                s[4 * f + 3] *= gg.w; dot += s[4 * f + 3] * kk[f].w; oq += s[4 * f + 3] * qq.w;
            }
            dot = part_sum<GD_PARTS>(dot);
            oq = part_sum<GD_PARTS>(oq);
            const float u = bs[tk] * (vs[tk * GD_CW + cl] - dot);
            // read-out of the updated state: (dS + k u^T)^T q = (dS)^T q + u (k.q)
            if (act && part == 0)
                obuf[((row0 + tk) * H + h) * (long)Dv + col] = oq + u * kqs[tk];
#pragma unroll
            for (int f = 0; f < F; ++f) {
                s[4 * f] += kk[f].x * u;
                s[4 * f + 1] += kk[f].y * u;
                s[4 * f + 2] += kk[f].z * u;
                s[4 * f + 3] += kk[f].w * u;
            }
        }
        __syncthreads();
    }
#undef GD_FETCH
    if (act) {
#pragma unroll
        for (int f = 0; f < F; ++f)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = (f * GD_PARTS + part) * 4 + e;
                if (row < D) st[row] = s[f * 4 + e];
            }
    }
}

// per-head RMS norm over the value channels, shared weight, sigmoid gate:
// one wave per (token, head); pad tokens produce zeros
template <typename T>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                     long gstride, const float* __restrict__ w, float eps,
                                     const int* __restrict__ pos, const int* __restrict__ seq,
                                     T* __restrict__ out, long ntok, int S, int H, int Dv,
                                     int gate_silu) {
    const int lane = threadIdx.x & (WAVE - 1);
    const long wid = (long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (wid >= ntok * H) return;
    const long tok = wid / H;
    const int h = wid % H;
    T* op = out + wid * Dv;
    if (pos[tok] < 0 || seq[tok / S] < 0) {
        for (int c = lane; c < Dv; c += WAVE) stf<T>(op + c, 0.f);
        return;
    }
    const float* ip = o + wid * Dv;
    float ss = 0.f;
    for (int c = lane; c < Dv; c += WAVE) { float v = ip[c]; ss += v * v; }
    const float inv = 1.f / sqrtf(wave_sum(ss) / Dv + eps);
    const T* gp = gate + tok * gstride + (long)h * Dv;
    for (int c = lane; c < Dv; c += WAVE) {
        const float gv = ldf<T>(gp + c);
        stf<T>(op + c, ip[c] * inv * w[c] * (gate_silu ? gv * sigmoidf_(gv) : sigmoidf_(gv)));
    }
}

// ------------------------------------------------------------- elementwise
template <typename T>
__global__ void softcap_kernel(const T* __restrict__ in, float* __restrict__ out, long n,
                               float cap) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (long)gridDim.x * blockDim.x)
        out[i] = cap * tanhf(ldf<T>(in + i) / cap);
}

// x += sa*a (+ sb*b), fp32 residual stream
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ x, const T* __restrict__ a, float sa,
                                    const T* __restrict__ b, float sb, long n) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (long)gridDim.x * blockDim.x) {
        float v = x[i] + sa * ldf<T>(a + i);
        if (b) v += sb * ldf<T>(b + i);
        x[i] = v;
    }
}

// out[r, c] = gelu_tanh(gu[r, c]) * gu[r, I + c]
template <typename T>
__global__ void gelu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, long rows, int I) {
    const long total = rows * I;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const long r = idx / I;
        const int c = idx % I;
        const float z = ldf<T>(gu + r * 2 * I + c);
        const float u = ldf<T>(gu + r * 2 * I + I + c);
        const float ge = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
        stf<T>(out + idx, ge * u);
    }
}

// 8 channels per thread, 16-byte accesses; rows on blockIdx.y (strided)
template <typename T>
__global__ void gelu_mul_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, long rows,
                                    int I) {
    const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (c >= I) return;
    for (long r = blockIdx.y; r < rows; r += gridDim.y) {
        float z[8], u[8], o[8];
        load8<T>(gu + r * 2 * I + c, z);
        load8<T>(gu + r * 2 * I + I + c, u);
#pragma unroll
        for (int e = 0; e < 8; ++e)
            o[e] = 0.5f * z[e] * (1.f + tanhf(0.7978845608028654f *
                                              (z[e] + 0.044715f * z[e] * z[e] * z[e]))) * u[e];
        T* op = out + r * I + c;
        if constexpr (sizeof(T) == 2) {
            uint32_t pk[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                pk[e] = (uint32_t)f2bf_rne(o[2 * e]) | ((uint32_t)f2bf_rne(o[2 * e + 1]) << 16);
            *reinterpret_cast<uint4*>(op) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
        } else {
            *reinterpret_cast<float4*>(op) = make_float4(o[0], o[1], o[2], o[3]);
            *reinterpret_cast<float4*>(op + 4) = make_float4(o[4], o[5], o[6], o[7]);
        }
    }
}


// ------------------------------------------------------------------ RMS norm
// x / sqrt(mean(x^2) + eps) * w (or * (1 + w)); one 256-thread workgroup per
// row, fp32 statistics; input and output rows may be strided slices. The *_vec
// variants move 8 channels per thread with 16-byte accesses (widths that are
// multiples of 8 on 16-byte aligned rows); the second pass re-reads the row
// from cache, so any width works.
template <typename T> DEV void store8(T* p, const float* v);
template <> DEV void store8<float>(float* p, const float* v) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
template <> DEV void store8<bf16>(bf16* p, const float* v) {
    uint32_t pk[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
        pk[e] = (uint32_t)f2bf_rne(v[2 * e]) | ((uint32_t)f2bf_rne(v[2 * e + 1]) << 16);
    *reinterpret_cast<uint4*>(p) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
}

template <typename TIn, typename TOut>
__global__ void __launch_bounds__(LN_THREADS)
rms_norm_vec_kernel(const TIn* __restrict__ x, long xs, const float* __restrict__ w, int one_plus,
                    float eps, TOut* __restrict__ out, long os, int C) {
    __shared__ float red[LN_THREADS / WAVE];
    const long row = blockIdx.x;
    const TIn* xr = x + row * xs;
    float s = 0.f;
    for (int c = threadIdx.x * 8; c < C; c += LN_THREADS * 8) {
        float v[8];
        load8<TIn>(xr + c, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) s += v[e] * v[e];
    }
    const float inv = 1.f / sqrtf(block_sum(s, red) / C + eps);
    TOut* o = out + row * os;
    const float add = one_plus ? 1.f : 0.f;
    for (int c = threadIdx.x * 8; c < C; c += LN_THREADS * 8) {
        float v[8], wv[8];
        load8<TIn>(xr + c, v);
        load8<float>(w + c, wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = v[e] * inv * (wv[e] + add);
        store8<TOut>(o + c, v);
    }
}

// post-norm residual step: stream[row] += rms_norm(v[row]) * (w | 1 + w) in fp32,
// v = y, or y + (sum of the row's `nc` coefficients) * extra (experts that pass
// their input through). `copy` (optional) receives the updated row in the next
// GEMM's input type, or, with `next_w`, the next sublayer's pre-norm
// rms_norm(updated row) * next_w: the row's new statistics come from the same
// pass that updates it.
template <typename TY, typename TC>
__global__ void __launch_bounds__(LN_THREADS)
add_rms_norm_vec_kernel(float* __restrict__ stream, const TY* __restrict__ y,
                        const float* __restrict__ w, int one_plus, float eps,
                        TC* __restrict__ copy, const TY* __restrict__ extra,
                        const float* __restrict__ coef, long cs, int nc,
                        const float* __restrict__ next_w, int C) {
    __shared__ float red[LN_THREADS / WAVE];
    const long row = blockIdx.x;
    const TY* yr = y + row * C;
    const TY* er = extra ? extra + row * C : nullptr;
    float cf = 0.f;
    if (er) for (int k = 0; k < nc; ++k) cf += coef[row * cs + k];
    float s = 0.f;
    for (int c = threadIdx.x * 8; c < C; c += LN_THREADS * 8) {
        float v[8];
        load8<TY>(yr + c, v);
        if (er) {
            float ev[8];
            load8<TY>(er + c, ev);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] += cf * ev[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) s += v[e] * v[e];
    }
    const float inv = 1.f / sqrtf(block_sum(s, red) / C + eps);
    const float add = one_plus ? 1.f : 0.f;
    float* xr = stream + row * C;
    float s2 = 0.f;
    for (int c = threadIdx.x * 8; c < C; c += LN_THREADS * 8) {
        float v[8], wv[8], xv[8];
        load8<TY>(yr + c, v);
        if (er) {
            float ev[8];
            load8<TY>(er + c, ev);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] += cf * ev[e];
        }
        load8<float>(w + c, wv);
        load8<float>(xr + c, xv);
#pragma unroll
        for (int e = 0; e < 8; ++e) { xv[e] += v[e] * inv * (wv[e] + add); s2 += xv[e] * xv[e]; }
        store8<float>(xr + c, xv);
        if (copy && !next_w) store8<TC>(copy + row * C + c, xv);
    }
    if (!copy || !next_w) return;                        // uniform
    __syncthreads();                                     // `red` is reused
    const float inv2 = 1.f / sqrtf(block_sum(s2, red) / C + eps);
    for (int c = threadIdx.x * 8; c < C; c += LN_THREADS * 8) {
        float xv[8], wv[8];
        load8<float>(xr + c, xv);                        // this thread's own stores
        load8<float>(next_w + c, wv);
#pragma unroll
        for (int e = 0; e < 8; ++e) xv[e] = xv[e] * inv2 * wv[e];
        store8<TC>(copy + row * C + c, xv);
    }
}

template <typename TIn, typename TOut>
__global__ void __launch_bounds__(LN_THREADS)
rms_norm_kernel(const TIn* __restrict__ x, long xs, const float* __restrict__ w, int one_plus,
                float eps, TOut* __restrict__ out, long os, int C) {
    __shared__ float red[LN_THREADS / WAVE];
    const long row = blockIdx.x;
    const TIn* xr = x + row * xs;
    float s = 0.f;
    for (int c = threadIdx.x; c < C; c += LN_THREADS) { const float v = ldf<TIn>(xr + c); s += v * v; }
    const float inv = 1.f / sqrtf(block_sum(s, red) / C + eps);
    TOut* o = out + row * os;
    const float add = one_plus ? 1.f : 0.f;
    for (int c = threadIdx.x; c < C; c += LN_THREADS)
        stf<TOut>(o + c, ldf<TIn>(xr + c) * inv * (w[c] + add));
}

// scalar form of add_rms_norm_vec_kernel (any width and alignment)
template <typename TY, typename TC>
__global__ void __launch_bounds__(LN_THREADS)
add_rms_norm_kernel(float* __restrict__ stream, const TY* __restrict__ y,
                    const float* __restrict__ w, int one_plus, float eps,
                    TC* __restrict__ copy, const TY* __restrict__ extra,
                    const float* __restrict__ coef, long cs, int nc,
                    const float* __restrict__ next_w, int C) {
    __shared__ float red[LN_THREADS / WAVE];
    const long row = blockIdx.x;
    const TY* yr = y + row * C;
    const TY* er = extra ? extra + row * C : nullptr;
    float cf = 0.f;
    if (er) for (int k = 0; k < nc; ++k) cf += coef[row * cs + k];
    float s = 0.f;
    for (int c = threadIdx.x; c < C; c += LN_THREADS) {
        const float v = ldf<TY>(yr + c) + (er ? cf * ldf<TY>(er + c) : 0.f);
        s += v * v;
    }
    const float inv = 1.f / sqrtf(block_sum(s, red) / C + eps);
    const float add = one_plus ? 1.f : 0.f;
    float* xr = stream + row * C;
    float s2 = 0.f;
    for (int c = threadIdx.x; c < C; c += LN_THREADS) {
        const float yv = ldf<TY>(yr + c) + (er ? cf * ldf<TY>(er + c) : 0.f);
        const float v = xr[c] + yv * inv * (w[c] + add);
        xr[c] = v;
        s2 += v * v;
        if (copy && !next_w) stf<TC>(copy + row * C + c, v);
    }
    if (!copy || !next_w) return;                        // uniform
    __syncthreads();
    const float inv2 = 1.f / sqrtf(block_sum(s2, red) / C + eps);
    for (int c = threadIdx.x; c < C; c += LN_THREADS)
        stf<TC>(copy + row * C + c, xr[c] * inv2 * next_w[c]);
}

// ---------------------------------------------------------- rotary positions
// pairs (2i, 2i+1) of the first 2*half channels of every head turn by
// p * inv_freq[i] (fp32 angle, full-range sincosf); the rest is copied.
// One thread per (token, head, channel pair or trailing channel).
template <typename TIn, typename TOut>
__global__ void rope_pairs_kernel(const TIn* __restrict__ x, long xt, long xh,
                                  TOut* __restrict__ out, long ot, long oh,
                                  const int* __restrict__ pos, const float* __restrict__ inv_freq,
                                  int half, long ntok, int N, int C) {
    const int per = half + (C - 2 * half);            // work items per head
    const long total = ntok * N * per;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int e = idx % per;
        const long th = idx / per;
        const int h = th % N;
        const long tok = th / N;
        const int p = pos[tok];
        const TIn* xp = x + tok * xt + (long)h * xh;
        TOut* op = out + tok * ot + (long)h * oh;
        if (e < half) {
            float a = ldf<TIn>(xp + 2 * e), b = ldf<TIn>(xp + 2 * e + 1);
            float sn, cs;
            sincosf((float)(p < 0 ? 0 : p) * inv_freq[e], &sn, &cs);
            stf<TOut>(op + 2 * e, a * cs - b * sn);
            stf<TOut>(op + 2 * e + 1, b * cs + a * sn);
        } else {
            const int c = 2 * half + (e - half);
            stf<TOut>(op + c, ldf<TIn>(xp + c));
        }
    }
}

// ------------------------------------------------------- clamped gated unit
// out[r, c] = g * sigmoid(alpha * g) * (u + 1), g = min(gu[r, c], limit),
// u = clamp(gu[r, I + c], -limit, limit)
DEV float clamped_glu_(float g, float u, float limit, float alpha) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * sigmoidf_(alpha * g) * (u + 1.f);
}

template <typename T>
__global__ void clamped_glu_kernel(const T* __restrict__ gu, T* __restrict__ out, long rows, int I,
                                   float limit, float alpha) {
    const long total = rows * I;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const long r = idx / I;
        const int c = idx % I;
        stf<T>(out + idx, clamped_glu_(ldf<T>(gu + r * 2 * I + c), ldf<T>(gu + r * 2 * I + I + c),
                                       limit, alpha));
    }
}

template <typename T>
__global__ void clamped_glu_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, long rows,
                                       int I, float limit, float alpha) {
    const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (c >= I) return;
    for (long r = blockIdx.y; r < rows; r += gridDim.y) {
        float z[8], u[8], o[8];
        load8<T>(gu + r * 2 * I + c, z);
        load8<T>(gu + r * 2 * I + I + c, u);
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = clamped_glu_(z[e], u[e], limit, alpha);
        T* op = out + r * I + c;
        if constexpr (sizeof(T) == 2) {
            uint32_t pk[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                pk[e] = (uint32_t)f2bf_rne(o[2 * e]) | ((uint32_t)f2bf_rne(o[2 * e + 1]) << 16);
            *reinterpret_cast<uint4*>(op) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
        } else {
            *reinterpret_cast<float4*>(op) = make_float4(o[0], o[1], o[2], o[3]);
            *reinterpret_cast<float4*>(op + 4) = make_float4(o[4], o[5], o[6], o[7]);
        }
    }
}

// ------------------------------------------- per-head norm + half-split rotary
// One wave per (token, head): RMS norm over the head's C channels with a weight
// shared by the heads (optional), then rotary positions on the first 2*half
// channels, channel i paired with channel i + half, angle pos * inv_freq[i],
// cos and sin times mscale (half = 0: none). Statistics and angles are fp32;
// the normed row goes through LDS so a lane can read its partner channel.
#define HN_WAVES 4
#define HN_MAXC 512

template <typename TIn, typename TOut>
__global__ void __launch_bounds__(HN_WAVES * WAVE)
head_norm_rope_kernel(const TIn* __restrict__ x, long xt, long xh, TOut* __restrict__ out,
                      const int* __restrict__ pos, const float* __restrict__ nw, float eps,
                      const float* __restrict__ inv_freq, int half, float mscale,
                      long ntok, int N, int C) {
    __shared__ float rows[HN_WAVES][HN_MAXC];
    const int lane = threadIdx.x & (WAVE - 1), wv = threadIdx.x / WAVE;
    const long id = (long)blockIdx.x * HN_WAVES + wv;
    if (id >= ntok * N) return;
    const long tok = id / N;
    const int hd = id % N;
    const int p = pos[tok];
    TOut* op = out + (tok * N + hd) * (long)C;
    if (p < 0) {
        for (int c = lane; c < C; c += WAVE) stf<TOut>(op + c, 0.f);
        return;
    }
    const TIn* xp = x + tok * xt + (long)hd * xh;
    float* row = rows[wv];
    float ss = 0.f;
    for (int c = lane; c < C; c += WAVE) {
        const float v = ldf<TIn>(xp + c);
        row[c] = v;
        ss += v * v;
    }
    if (nw) {
        const float inv = 1.f / sqrtf(wave_sum(ss) / C + eps);
        for (int c = lane; c < C; c += WAVE) row[c] = row[c] * inv * nw[c];
    }
    __builtin_amdgcn_wave_barrier();
    // a lane owns whole pairs: one sincos serves both channels
    for (int i = lane; i < half; i += WAVE) {
        float sn, cs;
        sincosf((float)p * inv_freq[i], &sn, &cs);
        sn *= mscale; cs *= mscale;
        const float u = row[i], w2 = row[i + half];
        stf<TOut>(op + i, u * cs - w2 * sn);
        stf<TOut>(op + i + half, w2 * cs + u * sn);
    }
    for (int c = 2 * half + lane; c < C; c += WAVE) stf<TOut>(op + c, row[c]);
}

// ----------------------------------------------- scalar-decay linear recurrence
// S_t = a_t S_{t-1} + k_t (w_t v_t)^T, o_t = S_t^T q_t (+ skip_h v_t), one scalar
// decay per head and token. Workgroup = (row, head, 16 value channels); the 16
// lanes of a channel split its key rows (lane p owns rows p*R .. p*R+R-1), the
// state sits in registers for the whole step and is read/written once. Tokens
// are staged through LDS in chunks of DS_TC (q, k, v, decay, step size), so
// global loads are coalesced and the serial loop reads only LDS.
// Decay: selective (dt projection + dt_bias, a_log: w = softplus(dt + bias),
// a = exp(-exp(a_log) w)) or fixed per head (head_decay: a = decay, w = 1).
//
// Long rows with few workgroups are cut into `nseg` segments of `seglen`
// tokens that run side by side; the recurrence is linear in the state, so
//   MODE 1: every segment scans from a ZERO state and leaves its end state E_c
//           and the product P_c of its decays in the workspace (no outputs);
//   decay_scan_link_kernel: start state of segment c, serially over the few
//           segments: S_c = P_{c-1} S_{c-1} + E_{c-1} (S_0 = the carried state);
//   MODE 2: every segment scans again from its true start state and writes
//           the outputs; the last one stores the carried state.
// MODE 0 is the plain single pass (decode steps, short portions, full batches).
#define DS_TC 16

template <typename T, typename TD, int R, int MODE>
__global__ void __launch_bounds__(256)
decay_scan_kernel(const T* __restrict__ q, long qs, const T* __restrict__ k, long ks,
                  const T* __restrict__ v, long vs, const TD* __restrict__ dt, long dts,
                  const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                  const float* __restrict__ head_decay, float k_scale,
                  const float* __restrict__ skip, float* __restrict__ state,
                  const int* __restrict__ pos, const int* __restrict__ seq,
                  const int* __restrict__ nvalid, float* __restrict__ out, int S, int H, int G,
                  int D, int Dv, float* __restrict__ ws, float* __restrict__ wdec, int nseg,
                  int seglen) {
    constexpr int DP = 16 * R;
    __shared__ __attribute__((aligned(16))) float sq[MODE == 1 ? 1 : DS_TC][DP], sk[DS_TC][DP];
    __shared__ float sv[DS_TC][16], sa[DS_TC], sw[DS_TC];
    const int b = blockIdx.z, h = blockIdx.y;
    const int sgi = MODE == 0 ? 0 : blockIdx.x % nseg;
    const int c0 = (MODE == 0 ? blockIdx.x : blockIdx.x / nseg) * 16;
    const int slot = seq[b];
    const int n = slot < 0 ? 0 : nvalid[b];
    if (n <= 0) return;                                   // uniform
    const int tid = threadIdx.x, part = tid & 15, cl = tid >> 4;
    const int c = c0 + cl;
    const bool cok = c < Dv;
    const int g = h / (H / G);
    const int p0 = pos[(long)b * S];
    const int tbeg = MODE == 0 ? 0 : min(n, sgi * seglen);
    const int tend = MODE == 0 ? n : min(n, tbeg + seglen);
    float* sp = state + (((long)slot * H + h) * Dv + (cok ? c : 0)) * (long)D;
    float* wp = MODE == 0 ? nullptr
        : ws + ((((long)b * nseg + sgi) * H + h) * Dv + (cok ? c : 0)) * (long)D;
    float st[R];
    const float* src = MODE == 0 ? (p0 > 0 ? sp : nullptr) : (MODE == 2 ? wp : nullptr);
    // a lane's rows are contiguous in memory too: 16-byte accesses when the
    // row length allows (every state row then starts on a 16-byte boundary)
    const bool v4 = (R % 4 == 0) && (D % 4 == 0);
    if (v4) {
#pragma unroll
        for (int r = 0; r < R; r += 4) {
            const int d = part * R + r;
            float4 s4 = make_float4(0.f, 0.f, 0.f, 0.f);
            if (cok && src && d < D) s4 = *reinterpret_cast<const float4*>(src + d);
            st[r] = s4.x; st[r + 1 < R ? r + 1 : r] = s4.y;
            st[r + 2 < R ? r + 2 : r] = s4.z; st[r + 3 < R ? r + 3 : r] = s4.w;
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int d = part * R + r;
            st[r] = (cok && src && d < D) ? src[d] : 0.f;
        }
    }
    const float skp = skip ? skip[h] : 0.f;
    float aprod = 1.f;
    for (int t0 = tbeg; t0 < tend; t0 += DS_TC) {
        const int cnt = min(DS_TC, tend - t0);
        __syncthreads();                                  // the previous chunk is consumed
        for (int idx = tid; idx < DS_TC * DP; idx += 256) {
            const int tt = idx / DP, d = idx % DP;
            float qv = 0.f, kv = 0.f;
            if (tt < cnt && d < D) {
                const long tok = (long)b * S + t0 + tt;
                if (MODE != 1) qv = ldf<T>(q + tok * qs + (long)g * D + d);
                kv = ldf<T>(k + tok * ks + (long)g * D + d) * k_scale;
            }
            if (MODE != 1) sq[tt][d] = qv;
            sk[tt][d] = kv;
        }
        {
            const int tt = tid >> 4, cc = tid & 15;       // 256 = DS_TC * 16
            float vv = 0.f;
            if (tt < cnt && c0 + cc < Dv)
                vv = ldf<T>(v + ((long)b * S + t0 + tt) * vs + (long)h * Dv + c0 + cc);
            sv[tt][cc] = vv;
        }
        if (tid < cnt) {
            float a, w = 1.f;
            if (dt) {
                w = softplusf_(ldf<TD>(dt + ((long)b * S + t0 + tid) * dts + h) + dt_bias[h]);
                a = expf(-expf(a_log[h]) * w);
            } else {
                a = head_decay[h];
            }
            sa[tid] = a;
            sw[tid] = w;
        }
        __syncthreads();
        for (int tt = 0; tt < cnt; ++tt) {
            const float a = sa[tt], xv = sv[tt][cl];
            const float wv = sw[tt] * xv;
            // a lane's key rows are contiguous: 16-byte LDS reads
            float kr[R], qr[R];
            if constexpr (R % 4 == 0) {
#pragma unroll
                for (int r = 0; r < R; r += 4) {
                    const float4 k4 = *reinterpret_cast<const float4*>(&sk[tt][part * R + r]);
                    kr[r] = k4.x; kr[r + 1] = k4.y; kr[r + 2] = k4.z; kr[r + 3] = k4.w;
                    if (MODE != 1) {
                        const float4 q4 = *reinterpret_cast<const float4*>(&sq[tt][part * R + r]);
                        qr[r] = q4.x; qr[r + 1] = q4.y; qr[r + 2] = q4.z; qr[r + 3] = q4.w;
                    }
                }
            } else {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    kr[r] = sk[tt][part * R + r];
                    if (MODE != 1) qr[r] = sq[tt][part * R + r];
                }
            }
            if (MODE == 1) {
                aprod *= a;
#pragma unroll
                for (int r = 0; r < R; ++r) st[r] = a * st[r] + kr[r] * wv;
            } else {
                float acc = 0.f;
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    st[r] = a * st[r] + kr[r] * wv;
                    acc += st[r] * qr[r];
                }
                acc += __shfl_xor(acc, 8, WAVE);
                acc += __shfl_xor(acc, 4, WAVE);
                acc += __shfl_xor(acc, 2, WAVE);
                acc += __shfl_xor(acc, 1, WAVE);
                if (part == 0 && cok)
                    out[(((long)b * S + t0 + tt) * H + h) * (long)Dv + c] = acc + skp * xv;
            }
        }
    }
    if (MODE == 1 && c0 == 0 && tid == 0) wdec[((long)b * nseg + sgi) * H + h] = aprod;
    float* dst = MODE == 1 ? wp : ((MODE == 0 || sgi == nseg - 1) ? sp : nullptr);
    if (cok && dst) {
        if (v4) {
#pragma unroll
            for (int r = 0; r < R; r += 4) {
                const int d = part * R + r;
                if (d < D)
                    *reinterpret_cast<float4*>(dst + d) = make_float4(
                        st[r], st[r + 1 < R ? r + 1 : r], st[r + 2 < R ? r + 2 : r],
                        st[r + 3 < R ? r + 3 : r]);
            }
        } else {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int d = part * R + r;
                if (d < D) dst[d] = st[r];
            }
        }
    }
}

// start states of the segments, in place over their end states (see above)
__global__ void decay_scan_link_kernel(float* __restrict__ ws, const float* __restrict__ wdec,
                                       const float* __restrict__ state,
                                       const int* __restrict__ pos, const int* __restrict__ seq,
                                       const int* __restrict__ nvalid, int B, int S, int H,
                                       long per_head, int nseg) {
    const long total = (long)B * H * per_head;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long)gridDim.x * blockDim.x) {
        const long e = i % per_head;
        const int h = (i / per_head) % H;
        const int b = i / (per_head * H);
        const int slot = seq[b];
        if (slot < 0 || nvalid[b] <= 0) continue;
        float s = pos[(long)b * S] > 0 ? state[((long)slot * H + h) * per_head + e] : 0.f;
        for (int c = 0; c < nseg; ++c) {
            float* p = ws + (((long)b * nseg + c) * H + h) * per_head + e;
            const float end = *p;
            *p = s;
            s = wdec[((long)b * nseg + c) * H + h] * s + end;
        }
    }
}

// ------------------------------------------------ grouped RMS norm with silu gate
// One wave per (row, group of C/groups channels): y (fp32) is multiplied by
// silu(gate) before the norm (gate_first) or after it; optional weight.
template <typename TG, typename TOut>
__global__ void group_gated_norm_kernel(const float* __restrict__ y, const TG* __restrict__ gate,
                                        long gs, const float* __restrict__ w, float eps,
                                        int groups, int gate_first, TOut* __restrict__ out,
                                        long rows, int C) {
    const int lane = threadIdx.x & (WAVE - 1);
    const long id = (long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (id >= rows * groups) return;
    const long row = id / groups;
    const int gi = id % groups, Cg = C / groups;
    const float* yp = y + row * C + (long)gi * Cg;
    const TG* gp = gate + row * gs + (long)gi * Cg;
    const float* wp = w ? w + (long)gi * Cg : nullptr;
    TOut* op = out + row * C + (long)gi * Cg;
    float ss = 0.f;
    for (int c = lane; c < Cg; c += WAVE) {
        float v = yp[c];
        if (gate_first) { const float gv = ldf<TG>(gp + c); v *= gv * sigmoidf_(gv); }
        ss += v * v;
    }
    const float inv = 1.f / sqrtf(wave_sum(ss) / Cg + eps);
    for (int c = lane; c < Cg; c += WAVE) {
        const float gv = ldf<TG>(gp + c);
        const float sg = gv * sigmoidf_(gv);
        float v = yp[c];
        if (gate_first) v *= sg;
        v *= inv;
        if (wp) v *= wp[c];
        if (!gate_first) v *= sg;
        stf<TOut>(op + c, v);
    }
}

// ------------------------------------------------------- group-limited router
// One wave per token: softmax over E logits (fp32), group score = best expert of
// the group, `keep` best groups stay, `top` best experts among them are chosen
// (ties: lowest index). Writes the dense (T, E + extra) weight row (zeros at
// unchosen experts, sigmoid gates in the extra columns), the chosen indices and
// their weights = score * scale (renormalised over the chosen first if asked).
// `corr` (E, or null) is added to the scores for the group ranking and the choice
// only.
// A row whose logits are not numbers (the garbage of a pad token) selects the
// first experts with weight zero: every index stays in range.
DEV void wave_argmax(float& v, int& i) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o, WAVE);
        const int oi = __shfl_xor(i, o, WAVE);
        if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
    }
}

#define RT_WAVES 4
// one wave: logits `lp` (E + extra, global or LDS) of a token -> its dense row
// `dp`, chosen indices `idx` and weights `wts`; `cand` is 2E + ngroups floats of
// LDS scratch
DEV void route_select_(const float* lp, int E, int extra, int top, int ngroups, int keep,
                       float scale, int normalize, const float* __restrict__ corr, float* cand,
                       float* __restrict__ dp, int* __restrict__ idx, float* __restrict__ wts,
                       int lane) {
    float* gsc = cand + E;
    float* sco = gsc + ngroups;                   // the uncorrected scores (the weights)
    float m = -INFINITY;
    for (int e = lane; e < E; e += WAVE) m = fmaxf(m, lp[e]);
    m = wave_max(m);
    float sum = 0.f;
    for (int e = lane; e < E; e += WAVE) { const float x = expf(lp[e] - m); cand[e] = x; sum += x; }
    sum = wave_sum(sum);
    const float rs = 1.f / sum;
    for (int e = lane; e < E; e += WAVE) {
        const float sc = cand[e] * rs;
        sco[e] = sc;
        cand[e] = corr ? sc + corr[e] : sc;       // the choice goes by the corrected score
        dp[e] = 0.f;
    }
    for (int x = lane; x < extra; x += WAVE) dp[E + x] = sigmoidf_(lp[E + x]);
    __builtin_amdgcn_wave_barrier();
    const int per = E / ngroups;
    if (ngroups > 1 && keep < ngroups) {
        for (int gi = lane; gi < ngroups; gi += WAVE) {
            float gm = -INFINITY;
            for (int j = 0; j < per; ++j) gm = fmaxf(gm, cand[gi * per + j]);
            gsc[gi] = gm;
        }
        __builtin_amdgcn_wave_barrier();
        for (int r = 0; r < keep; ++r) {
            float bv = -INFINITY; int bi = 0x7fffffff;
            for (int gi = lane; gi < ngroups; gi += WAVE) {
                const float x = gsc[gi];
                if (x < INFINITY && (x > bv)) { bv = x; bi = gi; }
            }
            wave_argmax(bv, bi);
            if ((unsigned)bi >= (unsigned)ngroups) bi = r;   // a row of NaNs compares false everywhere
            if (lane == 0) gsc[bi] = INFINITY;            // kept
            __builtin_amdgcn_wave_barrier();
        }
        for (int e = lane; e < E; e += WAVE) if (gsc[e / per] != INFINITY) cand[e] = -INFINITY;
        __builtin_amdgcn_wave_barrier();
    }
    float wsum = 0.f;
    float myw = 0.f; int myi = 0;                         // lane r keeps the r-th choice
    for (int r = 0; r < top; ++r) {
        float bv = -INFINITY; int bi = 0x7fffffff;
        for (int e = lane; e < E; e += WAVE) {
            const float x = cand[e];
            if (x > bv) { bv = x; bi = e; }
        }
        wave_argmax(bv, bi);
        if ((unsigned)bi >= (unsigned)E) { bi = r; bv = 0.f; }   // NaN row (a pad token): any valid index
        else bv = sco[bi];                                // the weight is the score itself
        if (lane == 0) cand[bi] = -INFINITY;
        if (lane == (r & (WAVE - 1))) {
            // more than 64 choices: flush the previous one first
            if (r >= WAVE) { idx[r - WAVE] = myi; wts[r - WAVE] = myw; }
            myw = bv; myi = bi;
        }
        wsum += bv;
        __builtin_amdgcn_wave_barrier();
    }
    const float f = normalize ? scale / wsum : scale;
    if (top <= WAVE) {
        if (lane < top) {
            idx[lane] = myi;
            wts[lane] = myw * f;
            dp[myi] = myw * f;
        }
    }
}

__global__ void __launch_bounds__(RT_WAVES * WAVE)
group_router_kernel(const float* __restrict__ logits, long ls, int E, int extra, int top,
                    int ngroups, int keep, float scale, int normalize,
                    const float* __restrict__ corr,
                    float* __restrict__ dense, int* __restrict__ idx, float* __restrict__ wts,
                    long T) {
    extern __shared__ float rsm[];                // per wave: E choice scores + ngroups + E scores
    const int lane = threadIdx.x & (WAVE - 1), wv = threadIdx.x / WAVE;
    const long t = (long)blockIdx.x * RT_WAVES + wv;
    if (t >= T) return;
    route_select_(logits + t * ls, E, extra, top, ngroups, keep, scale, normalize, corr,
                  rsm + (long)wv * (2 * E + ngroups), dense + t * (long)(E + extra),
                  idx + t * top, wts + t * top, lane);
}

// Steps of few tokens: the router's product and its selection in one launch. One
// workgroup per token. The E + extra rows of the fp32 router weight are taken
// eight at a time: a thread reads its 8 channels of the token's input (widened to
// fp32) once and the same channels of the eight rows, all loads independent; the
// eight partial dot products are summed over the wave and over the four waves
// through LDS. The logits meet in LDS and the first wave selects as above.
template <typename T>
__global__ void __launch_bounds__(RT_WAVES * WAVE)
router_fused_kernel(const T* __restrict__ x, long xs, const float* __restrict__ w, int W, int vec,
                    int E, int extra, int top, int ngroups, int keep, float scale, int normalize,
                    const float* __restrict__ corr, float* __restrict__ dense,
                    int* __restrict__ idx, float* __restrict__ wts) {
    extern __shared__ float rsm[];                // E + extra logits, then the selection scratch
    __shared__ float part[RT_WAVES][8];
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wv = tid / WAVE;
    const long t = blockIdx.x;
    const T* xr = x + t * xs;
    const int rows = E + extra;
    for (int e0 = 0; e0 < rows; e0 += 8) {
        float acc[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) acc[k] = 0.f;
        if (vec) {
            for (int c = tid * 8; c < W; c += RT_WAVES * WAVE * 8) {
                float xv[8];
                load8<T>(xr + c, xv);
                float wv8[8][8];                         // rows past the last repeat it
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    load8<float>(w + (long)min(e0 + k, rows - 1) * W + c, wv8[k]);
#pragma unroll
                for (int k = 0; k < 8; ++k)
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[k] += xv[j] * wv8[k][j];
            }
        } else {
            for (int c = tid; c < W; c += RT_WAVES * WAVE) {
                const float xv = ldf<T>(xr + c);
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (e0 + k < rows) acc[k] += xv * w[(long)(e0 + k) * W + c];
            }
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float v = wave_sum(acc[k]);
            if (lane == 0) part[wv][k] = v;
        }
        __syncthreads();
        if (tid < 8 && e0 + tid < rows) {
            float v = 0.f;
#pragma unroll
            for (int q = 0; q < RT_WAVES; ++q) v += part[q][tid];
            rsm[e0 + tid] = v;
        }
        __syncthreads();
    }
    if (wv != 0) return;
    route_select_(rsm, E, extra, top, ngroups, keep, scale, normalize, corr, rsm + E + extra,
                  dense + t * (long)(E + extra), idx + t * top, wts + t * top, lane);
}

// -------------------------------------------------- relu^2 times routing weight
// out[t, c] = relu(x[t, c])^2 * gates[t, min(c / ff, E)] (gates = null: times one)
template <typename T>
__global__ void relu2_scale_kernel(const T* __restrict__ x, const float* __restrict__ gates,
                                   int gcols, int ff, int E, T* __restrict__ out, long rows,
                                   int C) {
    const long total = rows * C;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long)gridDim.x * blockDim.x) {
        const long t = i / C;
        const int c = i % C;
        const int e = min(c / ff, E);
        const float v = fmaxf(ldf<T>(x + i), 0.f);
        stf<T>(out + i, v * v * (gates ? gates[t * gcols + e] : 1.f));
    }
}

template <typename T>
__global__ void relu2_scale_vec_kernel(const T* __restrict__ x, const float* __restrict__ gates,
                                       int gcols, int ff, int E, T* __restrict__ out, long rows,
                                       int C) {
    const int C8 = C / 8;
    const long total = rows * C8;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long)gridDim.x * blockDim.x) {
        const long t = i / C8;
        const int c = (i % C8) * 8;
        const float gw = gates ? gates[t * gcols + min(c / ff, E)] : 1.f;
        float v[8];
        load8<T>(x + t * C + c, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) { const float r = fmaxf(v[e], 0.f); v[e] = r * r * gw; }
        store8<T>(out + t * C + c, v);
    }
}

// --------------------------------- clamped gated units of stacked experts
// x (rows, 2C) = [gate | up] pre-activations of C = E*ff + shared columns.
// out[t, c] = glu(gate, up; limit) * gates[t, c / ff] for c < E*ff (an expert's
// columns, times the token's routing weight), glu(gate, up; shared_limit) for the
// rest (an always-on shared expert); glu = g sigmoid(alpha g) (u + 1) on the
// clamped pre-activations.
template <typename T>
__global__ void clamped_glu_scale_kernel(const T* __restrict__ x, const float* __restrict__ gates,
                                         long gs, int ff, int E, float limit, float slimit,
                                         float alpha, T* __restrict__ out, long rows, int C) {
    const long total = rows * C;
    const int ne = E * ff;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long)gridDim.x * blockDim.x) {
        const long t = i / C;
        const int c = i % C;
        const bool own = c < ne;
        const float gw = own ? gates[t * gs + c / ff] : 1.f;
        float o = 0.f;
        if (gw != 0.f)
            o = clamped_glu_(ldf<T>(x + t * 2 * C + c), ldf<T>(x + t * 2 * C + C + c),
                             own ? limit : slimit, alpha) * gw;
        stf<T>(out + i, o);
    }
}

template <typename T>
__global__ void clamped_glu_scale_vec_kernel(const T* __restrict__ x,
                                             const float* __restrict__ gates, long gs, int ff,
                                             int E, float limit, float slimit, float alpha,
                                             T* __restrict__ out, long rows, int C) {
    const int C8 = C / 8;
    const long total = rows * C8;
    const int ne = E * ff;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long)gridDim.x * blockDim.x) {
        const long t = i / C8;
        const int c = (i % C8) * 8;                      // ff % 8 == 0: one owner per 8 columns
        const bool own = c < ne;
        const float gw = own ? gates[t * gs + c / ff] : 1.f;
        float o[8];
        if (gw != 0.f) {                                 // an unchosen expert's columns are not read
            float g[8], u[8];
            load8<T>(x + t * 2 * C + c, g);
            load8<T>(x + t * 2 * C + C + c, u);
            const float lim = own ? limit : slimit;
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = clamped_glu_(g[e], u[e], lim, alpha) * gw;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = 0.f;
        }
        store8<T>(out + t * C + c, o);
    }
}

// y[t, c] *= sigmoid(gate[t, c]); gate rows may be a column slice (row stride gs)
template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ y, const T* __restrict__ gate, long gs,
                                    long rows, int C, int vec) {
    if (vec) {
        const int C8 = C / 8;
        const long total = rows * C8;
        for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
             i += (long)gridDim.x * blockDim.x) {
            const long t = i / C8;
            const int c = (i % C8) * 8;
            float v[8], g[8];
            load8<T>(y + t * C + c, v);
            load8<T>(gate + t * gs + c, g);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] *= sigmoidf_(g[e]);
            store8<T>(y + t * C + c, v);
        }
        return;
    }
    const long total = rows * C;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long)gridDim.x * blockDim.x) {
        const long t = i / C;
        const int c = i % C;
        stf<T>(y + i, ldf<T>(y + i) * sigmoidf_(ldf<T>(gate + t * gs + c)));
    }
}

// 16-byte variant for rows of up to LN_THREADS * 8 * NV channels: every term is
// read once and stays in registers between the statistics and the update
template <typename T, int NV>
__global__ void __launch_bounds__(LN_THREADS)
scaled_residual_vec_kernel(float* __restrict__ x, const T* __restrict__ y0,
                           const float* __restrict__ w0, int n0, const T* __restrict__ y1,
                           const float* __restrict__ w1, int n1, const T* __restrict__ y2,
                           const float* __restrict__ w2, int n2, float eps, int C) {
    __shared__ float red[3][LN_THREADS / WAVE];
    const long row = blockIdx.x;
    const T* ys[3] = {y0, y1, y2};
    const float* ws[3] = {w0, w1, w2};
    const int ns[3] = {n0, n1, n2};
    float val[3][NV][8];
    float ss[3] = {0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        if (!ys[i]) continue;                             // uniform
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int c = (j * LN_THREADS + threadIdx.x) * 8;
            if (c < C) {
                load8<T>(ys[i] + row * C + c, val[i][j]);
#pragma unroll
                for (int e = 0; e < 8; ++e) ss[i] += val[i][j][e] * val[i][j][e];
            }
        }
    }
    const int lane = threadIdx.x & (WAVE - 1), wv = threadIdx.x / WAVE;
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        const float t = wave_sum(ss[i]);
        if (lane == 0) red[i][wv] = t;
    }
    __syncthreads();
    float inv[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < LN_THREADS / WAVE; ++k) t += red[i][k];
        inv[i] = (ys[i] && ns[i]) ? 1.f / sqrtf(t / C + eps) : 1.f;
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int c = (j * LN_THREADS + threadIdx.x) * 8;
        if (c >= C) continue;
        float xv[8];
        load8<float>(x + row * C + c, xv);
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            if (!ys[i]) continue;
            float wv8[8];
            load8<float>(ws[i] + c, wv8);
#pragma unroll
            for (int e = 0; e < 8; ++e) xv[e] += val[i][j][e] * inv[i] * wv8[e];
        }
        st8<float>(x + row * C + c, xv);
    }
}

// ------------------------------------------- embedding + learned position rows
// stream[t, :] = float(emb[t, :]) + float(table[max(pos[t], 0), :])
template <typename T>
__global__ void embed_pos_kernel(const T* __restrict__ emb, const T* __restrict__ table,
                                 const int* __restrict__ pos, float* __restrict__ out,
                                 long ntok, int C, int rows_in_table) {
    const long total = ntok * C;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long)gridDim.x * blockDim.x) {
        const long t = i / C;
        const int c = i % C;
        int p = pos[t];
        p = p < 0 ? 0 : (p >= rows_in_table ? rows_in_table - 1 : p);
        out[i] = ldf<T>(emb + i) + ldf<T>(table + (long)p * C + c);
    }
}

// ------------------------------------- residual sum of weighted, optionally normed terms
// x[row] += sum_i f_i(y_i[row]) * w_i, f_i = RMS norm over the row or identity.
// One workgroup per row; statistics fp32.
template <typename T>
__global__ void __launch_bounds__(LN_THREADS)
scaled_residual_kernel(float* __restrict__ x, const T* __restrict__ y0,
                       const float* __restrict__ w0, int n0, const T* __restrict__ y1,
                       const float* __restrict__ w1, int n1, const T* __restrict__ y2,
                       const float* __restrict__ w2, int n2, float eps, int C) {
    __shared__ float red[LN_THREADS / WAVE];
    const long row = blockIdx.x;
    const T* ys[3] = {y0, y1, y2};
    const float* ws[3] = {w0, w1, w2};
    const int ns[3] = {n0, n1, n2};
    float inv[3] = {1.f, 1.f, 1.f};
    float ss[3] = {0.f, 0.f, 0.f};
    for (int c = threadIdx.x; c < C; c += LN_THREADS) {
#pragma unroll
        for (int i = 0; i < 3; ++i)
            if (ys[i] && ns[i]) { const float v = ldf<T>(ys[i] + row * C + c); ss[i] += v * v; }
    }
#pragma unroll
    for (int i = 0; i < 3; ++i)
        if (ys[i] && ns[i]) inv[i] = 1.f / sqrtf(block_sum(ss[i], red) / C + eps);   // uniform
    float* xr = x + row * C;
    for (int c = threadIdx.x; c < C; c += LN_THREADS) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < 3; ++i)
            if (ys[i]) acc += ldf<T>(ys[i] + row * C + c) * inv[i] * ws[i][c];
        xr[c] += acc;
    }
}

// =================================================================== C ABI
static inline int grid_for(long total, int block, int cap = 8192) {
    long g = (total + block - 1) / block;
    if (g < 1) g = 1;
    return (int)(g > cap ? cap : g);
}

extern "C" {

int nx_layer_norm(const float* x, const float* w, void* out, int out_bf16, long rows, int C,
                  float eps, hipStream_t st) {
    if (rows <= 0) return 0;
    dim3 grid((unsigned)rows), block(LN_THREADS);
    if (out_bf16) layer_norm_kernel<bf16><<<grid, block, 0, st>>>(x, w, (bf16*)out, rows, C, eps);
    else layer_norm_kernel<float><<<grid, block, 0, st>>>(x, w, (float*)out, rows, C, eps);
    return (int)hipGetLastError();
}

int nx_short_conv(const void* x, long xs, int x_bf16, const float* w, const float* tail,
                  const int* pos, const int* seq, const int* nvalid, void* y, int y_bf16, int B,
                  int S, int C, int taps, int act_silu, int residual, const float* bias,
                  hipStream_t st) {
    const long total = (long)B * S * C;
    if (total <= 0) return 0;
    {
        // tiled path: 8-channel groups with 16-byte accesses on every row
        const int esz = x_bf16 ? 2 : 4;
        const int tiles = (S + SC_TT - 1) / SC_TT;
        const bool ok = taps >= 2 && taps <= 4 && (C % 8) == 0 && ((xs * esz) % 16) == 0 &&
                        ((uintptr_t)x % 16) == 0 && ((uintptr_t)y % 16) == 0 &&
                        ((uintptr_t)tail % 16) == 0 && (long)B * tiles <= 65535 && S >= 8;
        if (ok) {
            dim3 gt((C / 8 + 127) / 128, (unsigned)(B * tiles)), bt(128);
#define SCT(TI, TO, TP) short_conv_tile_kernel<TI, TO, TP><<<gt, bt, 0, st>>>( \
        (const TI*)x, xs, w, tail, pos, seq, nvalid, (TO*)y, S, C, tiles, act_silu, residual, bias)
#define SCTT(TI, TO) do { if (taps == 2) SCT(TI, TO, 2); else if (taps == 3) SCT(TI, TO, 3); \
                          else SCT(TI, TO, 4); } while (0)
            if (x_bf16 && y_bf16) SCTT(bf16, bf16);
            else if (x_bf16) SCTT(bf16, float);
            else if (y_bf16) SCTT(float, bf16);
            else SCTT(float, float);
#undef SCTT
#undef SCT
            return (int)hipGetLastError();
        }
    }
    dim3 grid(grid_for(total, 256)), block(256);
#define SC(TI, TO) short_conv_kernel<TI, TO><<<grid, block, 0, st>>>( \
        (const TI*)x, xs, w, tail, pos, seq, (TO*)y, B, S, C, taps, act_silu, residual, bias)
    if (x_bf16 && y_bf16) SC(bf16, bf16);
    else if (x_bf16) SC(bf16, float);
    else if (y_bf16) SC(float, bf16);
    else SC(float, float);
#undef SC
    return (int)hipGetLastError();
}

int nx_short_conv_commit(const void* x, long xs, int x_bf16, float* tail, const int* pos,
                         const int* seq, const int* nvalid, int B, int S, int C, int R,
                         hipStream_t st) {
    const long total = (long)B * C;
    if (total <= 0 || R <= 0) return 0;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (x_bf16) short_conv_commit_kernel<bf16><<<grid, block, 0, st>>>(
        (const bf16*)x, xs, tail, pos, seq, nvalid, B, S, C, R);
    else short_conv_commit_kernel<float><<<grid, block, 0, st>>>(
        (const float*)x, xs, tail, pos, seq, nvalid, B, S, C, R);
    return (int)hipGetLastError();
}

int nx_paged_kv_write(void* kc, void* vc, const void* k, long kstride, const void* v,
                      long vstride, int is_bf16, const int* slots, long N, int GDk, int GDv,
                      long nslots, hipStream_t st) {
    const long total = N * (GDk + GDv);
    if (total <= 0) return 0;
    dim3 grid(grid_for(total, 256)), block(256);
    if (is_bf16) paged_kv_write_kernel<bf16><<<grid, block, 0, st>>>(
        (bf16*)kc, (bf16*)vc, (const bf16*)k, kstride, (const bf16*)v, vstride, slots, N, GDk,
        GDv, nslots);
    else paged_kv_write_kernel<float><<<grid, block, 0, st>>>(
        (float*)kc, (float*)vc, (const float*)k, kstride, (const float*)v, vstride, slots, N,
        GDk, GDv, nslots);
    return (int)hipGetLastError();
}

int nx_paged_attn(const void* q, long qstride, const void* kc, long ktok, long khead,
                  const void* vc, long vtok, long vhead, const int* pos, const int* seq,
                  const int* btab, int max_blocks, const float* r1, const float* r2,
                  const float* sink, const void* gate, long gstride, void* out, int io_bf16,
                  int out_bf16, int B, int S, int H, int G, int Dk, int Dv, int bsz,
                  float scale, int window, int keep, float cap, float qt_coef, int qt_every,
                  float* ws, int nks, int ghead, int cmask, hipStream_t st) {
    if ((long)B * S <= 0) return 0;
    if (Dv > WAVE * 8 || H % G != 0 || Dk <= 0 || Dv <= 0) return -1;
    if (!io_bf16 && out_bf16) return -2;
    if (r2 != nullptr && r1 == nullptr) return -4;
    if (cmask < 0 || window < 1) return -7;
    const int esz = io_bf16 ? 2 : 4;
    const int vecn = 16 / esz;                            // elements per 16-byte load
    const bool k_al = (Dk % 8) == 0 && (ktok % vecn) == 0 && (khead % vecn) == 0 &&
                      ((uintptr_t)kc % 16) == 0;
    const bool v_al = (Dv % 8) == 0 && (vtok % vecn) == 0 && (vhead % vecn) == 0 &&
                      ((uintptr_t)vc % 16) == 0;
    if (io_bf16 && out_bf16 && S == 1 && G == 1 && vc == kc && vtok == ktok && k_al && v_al &&
        !r1 && !gate && cap <= 0.f && qt_every <= 0 && keep == 0 && H >= 8 &&
        Dk <= 640 && (qstride % 8) == 0 && ((uintptr_t)q % 16) == 0) {
        // latent caches, single-token steps: one workgroup per token reads each
        // key row once and covers 512 value channels
        const int dkp = (Dk + 31) & ~31;
        const int nsplit = (Dv + 511) / 512, hch = (H + 15) / 16;
        if (nks < 1 || !ws) nks = 1;
        if (nks > 8) return -6;
        dim3 gl(S * nks, hch * nsplit, B), bl(256);
#define LD(DKV) do { \
            const size_t lsh = (size_t)(LD_KT * (DKV + 8) + 4 * LD_VW * (LD_KT + 8)) * 2; \
            static bool attr_set = false; \
            if (!attr_set) { \
                if (hipFuncSetAttribute((const void*)latent_decode_mfma_kernel<DKV>, \
                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lsh) != hipSuccess) return -5; \
                attr_set = true; \
            } \
            latent_decode_mfma_kernel<DKV><<<gl, bl, lsh, st>>>( \
                (const bf16*)q, qstride, (const bf16*)kc, ktok, pos, seq, btab, max_blocks, sink, \
                (bf16*)out, H, Dk, Dv, bsz, S, scale, nsplit, nks, ws, window, cmask); } while (0)
        if (dkp <= 128) LD(128);
        else if (dkp <= 256) LD(256);
        else if (dkp <= 384) LD(384);
        else if (dkp <= 576) LD(576);
        else LD(640);
#undef LD
        if (nks > 1) {
            const long waves = (long)B * S * H;
            latent_decode_merge_kernel<<<(unsigned)((waves + 3) / 4), 4 * WAVE, 0, st>>>(
                ws, sink, pos, seq, (bf16*)out, (long)B * S, S, H, Dv, nks);
        }
        return (int)hipGetLastError();
    }
    {
        // matrix-core path: bf16 steps with prompt portions (any head sizes in
        // multiples of 8: keys up to 640 wide, wide values split over
        // workgroups), and single-token steps of wide multi-query layers, whose
        // many heads per cache row fill the 16-row tiles
        const int rp = H / G;
        const bool rep_ok = rp <= MA_ROWS;       // rows beyond QT*rep stay idle
        const int dkp = (Dk + 31) & ~31, dvp = (Dv + 31) & ~31;
        const bool wide = dkp > 192 || dvp > 128;
        const bool dk_ok = dkp <= 640;
        const bool steps_ok = S > 1 || (wide && rp >= 8);
        if (io_bf16 && out_bf16 && steps_ok && rep_ok && dk_ok && k_al && v_al &&
            (qstride % 8) == 0 && ((uintptr_t)q % 16) == 0) {
            const int QTm = MA_ROWS / rp;
            const int nsplit = wide ? (Dv + 127) / 128 : 1;
            dim3 gm((S + QTm - 1) / QTm, G * nsplit, B), bm(256);
#define MA(DKV, DVV, KTV) paged_attn_mfma_kernel<DKV, DVV, KTV, (KTV == 32)><<<gm, bm, 0, st>>>( \
        (const bf16*)q, qstride, (const bf16*)kc, (const bf16*)vc, pos, seq, btab, max_blocks, \
        r1, r2, (const bf16*)gate, gstride, (bf16*)out, H, G, Dk, Dv, bsz, S, scale, window, \
        keep, QTm, ktok, khead, vtok, vhead, sink, cap, qt_coef, qt_every, nsplit, ghead, cmask)
#define MAV(DKV) do { if (dvp == 32) MA(DKV, 32, 64); else if (dvp == 64) MA(DKV, 64, 64); \
                      else if (dvp == 96) MA(DKV, 96, 64); else MA(DKV, 128, 64); } while (0)
            if (wide) {
                if (dkp <= 128) MA(128, 128, 64);
                else if (dkp <= 192) MA(192, 128, 64);
                else if (dkp <= 256) MA(256, 128, 32);
                else if (dkp <= 384) MA(384, 128, 32);
                else if (dkp <= 576) MA(576, 128, 32);
                else MA(640, 128, 32);
            }
            else if (dkp == 32) MAV(32);
            else if (dkp == 64) MAV(64);
            else if (dkp == 96) MAV(96);
            else if (dkp == 128) MAV(128);
            else MAV(192);
#undef MAV
#undef MA
            return (int)hipGetLastError();
        }
    }
    const bool dec = S == 1;                              // pure decode step
    const int NQ = dec ? 4 : 16, NW = dec ? 16 : 4;
    const int rep = H / G;
    const int HPW = rep < NQ ? rep : NQ;                  // query heads per workgroup
    const int QT = NQ / HPW;                              // tokens per workgroup
    const int chunks = (rep + HPW - 1) / HPW;
    const int DkP = (Dk + 7) & ~7;
    dim3 grid((S + QT - 1) / QT, G * chunks, B), block(NW * WAVE);
    // decode shape: 8 value channels per lane when they tile a wave evenly
    int lpr = 0;
    if (dec && v_al) {
        const int l = Dv / 8;
        if (l <= WAVE && (l & (l - 1)) == 0) lpr = l;
    }
    int pws = (lpr > 0 && NQ * Dv > WAVE * NQ) ? NQ * Dv : WAVE * NQ;
    long ptile = (long)NW * pws;
    const long marea = (long)(NW / 2) * NQ * (Dv + 2);
    size_t sh = (size_t)(NQ * DkP + (ptile > marea ? ptile : marea)) * sizeof(float);
    if (sh > 60 * 1024 && lpr > 0) {                      // wide values: scalar P.V
        lpr = 0;
        pws = WAVE * NQ;
        ptile = (long)NW * pws;
        sh = (size_t)(NQ * DkP + (ptile > marea ? ptile : marea)) * sizeof(float);
    }
    if (sh > 150 * 1024) return -3;
    const int kvec = k_al ? 1 : 0;
    // beyond the default 64 KB of dynamic LDS a kernel has to be told its limit
#define WA(T, TO, MR, Q, W) if (sh > 60 * 1024 && hipFuncSetAttribute( \
        (const void*)window_attn_kernel<T, TO, MR, Q, W>, \
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh) != hipSuccess) return -5; \
    window_attn_kernel<T, TO, MR, Q, W><<<grid, block, sh, st>>>( \
        (const T*)q, qstride, (const T*)kc, (const T*)vc, pos, seq, btab, max_blocks, r1, r2, \
        (const T*)gate, gstride, (TO*)out, H, G, Dk, Dv, bsz, S, scale, window, keep, HPW, QT, \
        chunks, lpr, pws, ktok, khead, vtok, vhead, kvec, sink, cap, qt_coef, qt_every, ghead, \
        cmask)
#define WAS(T, TO, MR) do { if (dec) { WA(T, TO, MR, 4, 16); } else { WA(T, TO, MR, 16, 4); } } while (0)
#define WAM(T, TO) do { if (Dv <= 2 * WAVE) WAS(T, TO, 2); else if (Dv <= 4 * WAVE) WAS(T, TO, 4); \
                        else WAS(T, TO, 8); } while (0)
    if (io_bf16 && out_bf16) WAM(bf16, bf16);
    else if (io_bf16) WAM(bf16, float);
    else WAM(float, float);
#undef WAM
#undef WAS
#undef WA
    return (int)hipGetLastError();
}

int nx_gated_delta(const float* qkv, long cstride, const void* beta, long bstride, const void* a,
                   long astride, const void* gate, long gstride, const float* dt_bias,
                   const float* a_log, const float* norm_w, float eps, float* state,
                   const int* pos, const int* seq, const int* nvalid, float* prep, long PS,
                   float* obuf, void* out, int in_bf16, int B, int S, int H, int G, int D,
                   int Dv, int per_head, int gate_silu, hipStream_t st) {
    if (B <= 0 || S <= 0) return 0;
    if (D > 256 || H % G != 0 || PS < (long)(2 * G + H) * D + H + G) return -1;
    const long ntok = (long)B * S;
    {
        const long waves = ntok * (2 * G + H);
        dim3 g0((unsigned)((waves + 3) / 4)), b0(4 * WAVE);
        if (in_bf16) delta_prep_kernel<bf16><<<g0, b0, 0, st>>>(
            qkv, cstride, (const bf16*)beta, bstride, (const bf16*)a, astride, dt_bias, a_log,
            pos, seq, prep, PS, ntok, S, H, G, D, per_head);
        else delta_prep_kernel<float><<<g0, b0, 0, st>>>(
            qkv, cstride, (const float*)beta, bstride, (const float*)a, astride, dt_bias, a_log,
            pos, seq, prep, PS, ntok, S, H, G, D, per_head);
        int rc = (int)hipGetLastError();
        if (rc) return rc;
    }
    const int parts = D <= 32 ? 8 : 16;
    const int cw = GD_THREADS / parts;
    dim3 grid((Dv + cw - 1) / cw, H, B), block(GD_THREADS);
#define GD(DKV, TCV, PV) gated_delta_kernel<DKV, TCV, PV><<<grid, block, 0, st>>>( \
        qkv, cstride, prep, PS, state, pos, seq, nvalid, obuf, S, H, G, D, Dv)
    if (D <= 32) GD(32, 16, 8);
    else if (D <= 64) GD(64, 16, 16);
    else if (D <= 128) GD(128, 16, 16);
    else GD(256, 8, 16);
#undef GD
    int rc = (int)hipGetLastError();
    if (rc) return rc;
    const long waves = ntok * H;
    dim3 g2((unsigned)((waves + 3) / 4)), b2(4 * WAVE);
    if (in_bf16) gated_rmsnorm_kernel<bf16><<<g2, b2, 0, st>>>(
        obuf, (const bf16*)gate, gstride, norm_w, eps, pos, seq, (bf16*)out, ntok, S, H, Dv,
        gate_silu);
    else gated_rmsnorm_kernel<float><<<g2, b2, 0, st>>>(
        obuf, (const float*)gate, gstride, norm_w, eps, pos, seq, (float*)out, ntok, S, H, Dv,
        gate_silu);
    return (int)hipGetLastError();
}

int nx_softcap(const void* in, int in_bf16, float* out, long n, float cap, hipStream_t st) {
    if (n <= 0) return 0;
    dim3 grid(grid_for(n, 256)), block(256);
    if (in_bf16) softcap_kernel<bf16><<<grid, block, 0, st>>>((const bf16*)in, out, n, cap);
    else softcap_kernel<float><<<grid, block, 0, st>>>((const float*)in, out, n, cap);
    return (int)hipGetLastError();
}

int nx_residual_add(float* x, const void* a, float sa, const void* b, float sb, int is_bf16,
                    long n, hipStream_t st) {
    if (n <= 0) return 0;
    dim3 grid(grid_for(n, 256)), block(256);
    if (is_bf16) residual_add_kernel<bf16><<<grid, block, 0, st>>>(
        x, (const bf16*)a, sa, (const bf16*)b, sb, n);
    else residual_add_kernel<float><<<grid, block, 0, st>>>(
        x, (const float*)a, sa, (const float*)b, sb, n);
    return (int)hipGetLastError();
}

int nx_gelu_mul(const void* gu, void* out, int is_bf16, long rows, int I, hipStream_t st) {
    if (rows <= 0) return 0;
    if ((I % 8) == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)out % 16) == 0) {
        dim3 gv((I / 8 + 255) / 256, (unsigned)(rows > 32768 ? 32768 : rows)), bv(256);
        if (is_bf16) gelu_mul_vec_kernel<bf16><<<gv, bv, 0, st>>>((const bf16*)gu, (bf16*)out, rows, I);
        else gelu_mul_vec_kernel<float><<<gv, bv, 0, st>>>((const float*)gu, (float*)out, rows, I);
        return (int)hipGetLastError();
    }
    dim3 grid(grid_for(rows * I, 256)), block(256);
    if (is_bf16) gelu_mul_kernel<bf16><<<grid, block, 0, st>>>((const bf16*)gu, (bf16*)out, rows, I);
    else gelu_mul_kernel<float><<<grid, block, 0, st>>>((const float*)gu, (float*)out, rows, I);
    return (int)hipGetLastError();
}

int nx_rms_norm(const void* x, long xs, int x_bf16, const float* w, int one_plus, float eps,
                void* out, long os, int out_bf16, long rows, int C, hipStream_t st) {
    if (rows <= 0) return 0;
    dim3 grid((unsigned)rows), block(LN_THREADS);
    const int xe = x_bf16 ? 2 : 4, oe = out_bf16 ? 2 : 4;
    const bool vec = (C % 8) == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                     ((xs * xe) % 16) == 0 && ((os * oe) % 16) == 0 && ((uintptr_t)w % 16) == 0;
#define RN(TI, TO) do { if (vec) rms_norm_vec_kernel<TI, TO><<<grid, block, 0, st>>>( \
        (const TI*)x, xs, w, one_plus, eps, (TO*)out, os, C); \
    else rms_norm_kernel<TI, TO><<<grid, block, 0, st>>>( \
        (const TI*)x, xs, w, one_plus, eps, (TO*)out, os, C); } while (0)
    if (x_bf16 && out_bf16) RN(bf16, bf16);
    else if (x_bf16) RN(bf16, float);
    else if (out_bf16) RN(float, bf16);
    else RN(float, float);
#undef RN
    return (int)hipGetLastError();
}

int nx_add_rms_norm(float* stream, const void* y, int y_bf16, const float* w, int one_plus,
                    float eps, void* copy, int copy_bf16, const void* extra, const float* coef,
                    long cs, int nc, const float* next_w, long rows, int C, hipStream_t st) {
    if (rows <= 0) return 0;
    if ((extra == nullptr) != (coef == nullptr)) return -1;
    dim3 grid((unsigned)rows), block(LN_THREADS);
    const bool vec = (C % 8) == 0 && ((uintptr_t)stream % 16) == 0 && ((uintptr_t)y % 16) == 0 &&
                     ((uintptr_t)copy % 16) == 0 && ((uintptr_t)w % 16) == 0 &&
                     ((uintptr_t)extra % 16) == 0 && ((uintptr_t)next_w % 16) == 0;
#define ARN(K, TY, TC) K<TY, TC><<<grid, block, 0, st>>>(stream, (const TY*)y, w, one_plus, eps, \
        (TC*)copy, (const TY*)extra, coef, cs, nc, next_w, C)
#define ARN2(K) do { if (y_bf16 && copy_bf16) ARN(K, bf16, bf16); else if (y_bf16) ARN(K, bf16, float); \
                     else if (copy_bf16) ARN(K, float, bf16); else ARN(K, float, float); } while (0)
    if (vec) ARN2(add_rms_norm_vec_kernel);
    else ARN2(add_rms_norm_kernel);
#undef ARN2
#undef ARN
    return (int)hipGetLastError();
}

int nx_rope_pairs(const void* x, long xt, long xh, int x_bf16, void* out, long ot, long oh,
                  int out_bf16, const int* pos, const float* inv_freq, int half, long ntok,
                  int N, int C, hipStream_t st) {
    const long total = ntok * N * (C - half);
    if (total <= 0) return 0;
    if (2 * half > C) return -1;
    dim3 grid(grid_for(total, 256)), block(256);
#define RP(TI, TO) rope_pairs_kernel<TI, TO><<<grid, block, 0, st>>>( \
        (const TI*)x, xt, xh, (TO*)out, ot, oh, pos, inv_freq, half, ntok, N, C)
    if (x_bf16 && out_bf16) RP(bf16, bf16);
    else if (x_bf16) RP(bf16, float);
    else if (out_bf16) RP(float, bf16);
    else RP(float, float);
#undef RP
    return (int)hipGetLastError();
}

int nx_clamped_glu(const void* gu, void* out, int is_bf16, long rows, int I, float limit,
                   float alpha, hipStream_t st) {
    if (rows <= 0) return 0;
    if ((I % 8) == 0 && ((uintptr_t)gu % 16) == 0 && ((uintptr_t)out % 16) == 0) {
        dim3 gv((I / 8 + 255) / 256, (unsigned)(rows > 32768 ? 32768 : rows)), bv(256);
        if (is_bf16) clamped_glu_vec_kernel<bf16><<<gv, bv, 0, st>>>(
            (const bf16*)gu, (bf16*)out, rows, I, limit, alpha);
        else clamped_glu_vec_kernel<float><<<gv, bv, 0, st>>>(
            (const float*)gu, (float*)out, rows, I, limit, alpha);
        return (int)hipGetLastError();
    }
    dim3 grid(grid_for(rows * I, 256)), block(256);
    if (is_bf16) clamped_glu_kernel<bf16><<<grid, block, 0, st>>>(
        (const bf16*)gu, (bf16*)out, rows, I, limit, alpha);
    else clamped_glu_kernel<float><<<grid, block, 0, st>>>(
        (const float*)gu, (float*)out, rows, I, limit, alpha);
    return (int)hipGetLastError();
}

int nx_head_norm_rope(const void* x, long xt, long xh, int x_bf16, void* out, int out_bf16,
                      const int* pos, const float* nw, float eps, const float* inv_freq,
                      int half, float mscale, long ntok, int N, int C, hipStream_t st) {
    if (ntok * N <= 0) return 0;
    if (C > HN_MAXC || 2 * half > C || (half > 0 && !inv_freq)) return -1;
    const long waves = ntok * N;
    dim3 grid((unsigned)((waves + HN_WAVES - 1) / HN_WAVES)), block(HN_WAVES * WAVE);
#define HN(TI, TO) head_norm_rope_kernel<TI, TO><<<grid, block, 0, st>>>( \
        (const TI*)x, xt, xh, (TO*)out, pos, nw, eps, inv_freq, half, mscale, ntok, N, C)
    if (x_bf16 && out_bf16) HN(bf16, bf16);
    else if (x_bf16) HN(bf16, float);
    else if (out_bf16) HN(float, bf16);
    else HN(float, float);
#undef HN
    return (int)hipGetLastError();
}

int nx_decay_scan(const void* q, long qs, const void* k, long ks, const void* v, long vs,
                  int in_bf16, const void* dt, long dts, int dt_bf16, const float* dt_bias,
                  const float* a_log, const float* head_decay, float k_scale, const float* skip,
                  float* state, const int* pos, const int* seq, const int* nvalid, float* out,
                  int B, int S, int H, int G, int D, int Dv, float* ws, float* wdec, int nseg,
                  int seglen, hipStream_t st) {
    if ((long)B * S <= 0) return 0;
    if (D <= 0 || Dv <= 0 || G <= 0 || H % G != 0 || D > 256) return -1;
    if ((dt == nullptr) == (head_decay == nullptr)) return -2;
    if (dt && (!dt_bias || !a_log)) return -2;
    if (H > 65535 || B > 65535) return -3;
    // the kernel reads state rows 16 bytes at a time when dim % 4 == 0
    if (((uintptr_t)state % 16) != 0 || ((uintptr_t)ws % 16) != 0) return -5;
    if (nseg < 1 || (nseg > 1 && (!ws || !wdec || seglen <= 0 || (long)nseg * seglen < S)))
        return -4;
    const int cb = (Dv + 15) / 16;
    dim3 grid(cb * nseg, H, B), block(256);
#define DSK(T, TD, RV, MD) decay_scan_kernel<T, TD, RV, MD><<<grid, block, 0, st>>>( \
        (const T*)q, qs, (const T*)k, ks, (const T*)v, vs, (const TD*)dt, dts, dt_bias, a_log, \
        head_decay, k_scale, skip, state, pos, seq, nvalid, out, S, H, G, D, Dv, ws, wdec, nseg, \
        seglen)
#define DSR(T, TD, MD) do { if (D <= 16) DSK(T, TD, 1, MD); else if (D <= 32) DSK(T, TD, 2, MD); \
        else if (D <= 64) DSK(T, TD, 4, MD); else if (D <= 128) DSK(T, TD, 8, MD); \
        else DSK(T, TD, 16, MD); } while (0)
#define DST(MD) do { \
        if (in_bf16) { if (dt_bf16) DSR(bf16, bf16, MD); else DSR(bf16, float, MD); } \
        else { if (dt_bf16) DSR(float, bf16, MD); else DSR(float, float, MD); } } while (0)
    if (nseg == 1) {
        DST(0);
    } else {
        DST(1);
        const long per_head = (long)Dv * D;
        decay_scan_link_kernel<<<grid_for((long)B * H * per_head, 256), 256, 0, st>>>(
            ws, wdec, state, pos, seq, nvalid, B, S, H, per_head, nseg);
        DST(2);
    }
#undef DST
#undef DSR
#undef DSK
    return (int)hipGetLastError();
}

int nx_group_gated_norm(const float* y, const void* gate, long gs, int gate_bf16, const float* w,
                        float eps, int groups, int gate_first, void* out, int out_bf16,
                        long rows, int C, hipStream_t st) {
    if (rows <= 0) return 0;
    if (groups <= 0 || C % groups != 0) return -1;
    const long waves = rows * groups;
    dim3 grid((unsigned)((waves + 3) / 4)), block(4 * WAVE);
#define GN(TG, TO) group_gated_norm_kernel<TG, TO><<<grid, block, 0, st>>>( \
        y, (const TG*)gate, gs, w, eps, groups, gate_first, (TO*)out, rows, C)
    if (gate_bf16 && out_bf16) GN(bf16, bf16);
    else if (gate_bf16) GN(bf16, float);
    else if (out_bf16) GN(float, bf16);
    else GN(float, float);
#undef GN
    return (int)hipGetLastError();
}

int nx_group_router(const float* logits, long ls, int E, int extra, int top, int ngroups,
                    int keep, float scale, int normalize, const float* corr, float* dense,
                    int* idx, float* wts, long T, hipStream_t st) {
    if (T <= 0) return 0;
    if (E <= 0 || top <= 0 || top > E || top > WAVE || ngroups <= 0 || E % ngroups != 0 ||
        keep <= 0 || keep > ngroups || (long)top > (long)(E / ngroups) * keep) return -1;
    const size_t sh = (size_t)RT_WAVES * (2 * E + ngroups) * sizeof(float);
    if (sh > 60 * 1024) return -2;
    dim3 grid((unsigned)((T + RT_WAVES - 1) / RT_WAVES)), block(RT_WAVES * WAVE);
    group_router_kernel<<<grid, block, sh, st>>>(logits, ls, E, extra, top, ngroups, keep, scale,
                                                 normalize, corr, dense, idx, wts, T);
    return (int)hipGetLastError();
}

int nx_router_fused(const void* x, long xs, int x_bf16, const float* w, int W, int E, int extra,
                    int top, int ngroups, int keep, float scale, int normalize, const float* corr,
                    float* dense, int* idx, float* wts, long T, hipStream_t st) {
    if (T <= 0) return 0;
    if (E <= 0 || top <= 0 || top > E || top > WAVE || ngroups <= 0 || E % ngroups != 0 ||
        keep <= 0 || keep > ngroups || (long)top > (long)(E / ngroups) * keep || W <= 0) return -1;
    const size_t sh = (size_t)(3 * E + extra + ngroups) * sizeof(float);
    if (sh > 60 * 1024) return -2;
    const int vecn = x_bf16 ? 8 : 4;
    const int vec = (W % 8) == 0 && (xs % vecn) == 0 && ((uintptr_t)x % 16) == 0 &&
                    ((uintptr_t)w % 16) == 0;
    dim3 grid((unsigned)T), block(RT_WAVES * WAVE);
    if (x_bf16) router_fused_kernel<bf16><<<grid, block, sh, st>>>(
        (const bf16*)x, xs, w, W, vec, E, extra, top, ngroups, keep, scale, normalize, corr, dense,
        idx, wts);
    else router_fused_kernel<float><<<grid, block, sh, st>>>(
        (const float*)x, xs, w, W, vec, E, extra, top, ngroups, keep, scale, normalize, corr, dense,
        idx, wts);
    return (int)hipGetLastError();
}

int nx_latent_row(const void* x, long xs, int is_bf16, const float* w, float eps,
                  const float* inv_freq, int half, const int* pos, const int* slots, void* cache,
                  long nslots, void* row, long rs, long ntok, int C, int R, hipStream_t st) {
    if (ntok <= 0) return 0;
    if (C <= 0 || R < 0 || 2 * half > R || (half > 0 && !inv_freq)) return -1;
    dim3 grid((unsigned)((ntok + 3) / 4)), block(4 * WAVE);
    if (is_bf16) latent_row_kernel<bf16><<<grid, block, 0, st>>>(
        (const bf16*)x, xs, w, eps, inv_freq, half, pos, slots, (bf16*)cache, nslots, (bf16*)row,
        rs, ntok, C, R);
    else latent_row_kernel<float><<<grid, block, 0, st>>>(
        (const float*)x, xs, w, eps, inv_freq, half, pos, slots, (float*)cache, nslots,
        (float*)row, rs, ntok, C, R);
    return (int)hipGetLastError();
}

int nx_relu2_scale(const void* x, int is_bf16, const float* gates, int gcols, int ff, int E,
                   void* out, long rows, int C, hipStream_t st) {
    if (rows * C <= 0) return 0;
    if (ff <= 0 || (gates && (gcols < E || (C > E * ff && gcols < E + 1)))) return -1;
    const int esz = is_bf16 ? 2 : 4;
    const bool vec = (C % 8) == 0 && (ff % 8) == 0 && ((uintptr_t)x % 16) == 0 &&
                     ((uintptr_t)out % 16) == 0 && esz > 0;
    if (vec) {
        dim3 grid(grid_for(rows * (C / 8), 256)), block(256);
        if (is_bf16) relu2_scale_vec_kernel<bf16><<<grid, block, 0, st>>>(
            (const bf16*)x, gates, gcols, ff, E, (bf16*)out, rows, C);
        else relu2_scale_vec_kernel<float><<<grid, block, 0, st>>>(
            (const float*)x, gates, gcols, ff, E, (float*)out, rows, C);
    } else {
        dim3 grid(grid_for(rows * C, 256)), block(256);
        if (is_bf16) relu2_scale_kernel<bf16><<<grid, block, 0, st>>>(
            (const bf16*)x, gates, gcols, ff, E, (bf16*)out, rows, C);
        else relu2_scale_kernel<float><<<grid, block, 0, st>>>(
            (const float*)x, gates, gcols, ff, E, (float*)out, rows, C);
    }
    return (int)hipGetLastError();
}

int nx_clamped_glu_scale(const void* x, int is_bf16, const float* gates, long gs, int ff, int E,
                         float limit, float slimit, float alpha, void* out, long rows, int C,
                         hipStream_t st) {
    if (rows * C <= 0) return 0;
    if (E < 0 || (E > 0 && (ff <= 0 || !gates)) || (long)E * ff > C) return -1;
    if (E == 0) ff = 8;
    const bool vec = (C % 8) == 0 && (ff % 8) == 0 && ((uintptr_t)x % 16) == 0 &&
                     ((uintptr_t)out % 16) == 0;
    if (vec) {
        dim3 grid(grid_for(rows * (C / 8), 256)), block(256);
        if (is_bf16) clamped_glu_scale_vec_kernel<bf16><<<grid, block, 0, st>>>(
            (const bf16*)x, gates, gs, ff, E, limit, slimit, alpha, (bf16*)out, rows, C);
        else clamped_glu_scale_vec_kernel<float><<<grid, block, 0, st>>>(
            (const float*)x, gates, gs, ff, E, limit, slimit, alpha, (float*)out, rows, C);
    } else {
        dim3 grid(grid_for(rows * C, 256)), block(256);
        if (is_bf16) clamped_glu_scale_kernel<bf16><<<grid, block, 0, st>>>(
            (const bf16*)x, gates, gs, ff, E, limit, slimit, alpha, (bf16*)out, rows, C);
        else clamped_glu_scale_kernel<float><<<grid, block, 0, st>>>(
            (const float*)x, gates, gs, ff, E, limit, slimit, alpha, (float*)out, rows, C);
    }
    return (int)hipGetLastError();
}

int nx_sigmoid_gate(void* y, const void* gate, long gs, int is_bf16, long rows, int C,
                    hipStream_t st) {
    if (rows * C <= 0) return 0;
    const int vecn = is_bf16 ? 8 : 4;                     // elements per 16 bytes
    const int vec = (C % 8) == 0 && (gs % vecn) == 0 && ((uintptr_t)y % 16) == 0 &&
                    ((uintptr_t)gate % 16) == 0;
    dim3 grid(grid_for(vec ? rows * (C / 8) : rows * C, 256)), block(256);
    if (is_bf16) sigmoid_gate_kernel<bf16><<<grid, block, 0, st>>>(
        (bf16*)y, (const bf16*)gate, gs, rows, C, vec);
    else sigmoid_gate_kernel<float><<<grid, block, 0, st>>>(
        (float*)y, (const float*)gate, gs, rows, C, vec);
    return (int)hipGetLastError();
}

int nx_scaled_residual(float* x, const void* y0, const float* w0, int n0, const void* y1,
                       const float* w1, int n1, const void* y2, const float* w2, int n2,
                       int is_bf16, float eps, long rows, int C, hipStream_t st) {
    if (rows <= 0) return 0;
    if (!y0 || !w0 || (y1 && !w1) || (y2 && !w2)) return -1;
    dim3 grid((unsigned)rows), block(LN_THREADS);
    const bool al = (C % 8) == 0 && C <= LN_THREADS * 8 * 4 && ((uintptr_t)x % 16) == 0 &&
        ((uintptr_t)y0 % 16) == 0 && ((uintptr_t)y1 % 16) == 0 && ((uintptr_t)y2 % 16) == 0 &&
        ((uintptr_t)w0 % 16) == 0 && ((uintptr_t)w1 % 16) == 0 && ((uintptr_t)w2 % 16) == 0;
    if (al) {
#define SRV(T, NVV) scaled_residual_vec_kernel<T, NVV><<<grid, block, 0, st>>>( \
        x, (const T*)y0, w0, n0, (const T*)y1, w1, n1, (const T*)y2, w2, n2, eps, C)
#define SRN(T) do { if (C <= LN_THREADS * 8) SRV(T, 1); else if (C <= LN_THREADS * 16) SRV(T, 2); \
                    else SRV(T, 4); } while (0)
        if (is_bf16) SRN(bf16); else SRN(float);
#undef SRN
#undef SRV
        return (int)hipGetLastError();
    }
    if (is_bf16) scaled_residual_kernel<bf16><<<grid, block, 0, st>>>(
        x, (const bf16*)y0, w0, n0, (const bf16*)y1, w1, n1, (const bf16*)y2, w2, n2, eps, C);
    else scaled_residual_kernel<float><<<grid, block, 0, st>>>(
        x, (const float*)y0, w0, n0, (const float*)y1, w1, n1, (const float*)y2, w2, n2, eps, C);
    return (int)hipGetLastError();
}

int nx_embed_pos(const void* emb, const void* table, int is_bf16, const int* pos, float* out,
                 long ntok, int C, int rows_in_table, hipStream_t st) {
    if (ntok * C <= 0) return 0;
    if (rows_in_table <= 0) return -1;
    dim3 grid(grid_for(ntok * C, 256)), block(256);
    if (is_bf16) embed_pos_kernel<bf16><<<grid, block, 0, st>>>(
        (const bf16*)emb, (const bf16*)table, pos, out, ntok, C, rows_in_table);
    else embed_pos_kernel<float><<<grid, block, 0, st>>>(
        (const float*)emb, (const float*)table, pos, out, ntok, C, rows_in_table);
    return (int)hipGetLastError();
}

}  // extern "C"
