// Kernels of decoders with a real-gated diagonal recurrence, rotated values and pooled blocks
// behind an attention window, and capped routed experts:
//   half_rope_store         q, k turned in half-split pairs (first `dims` entries), values turned
//                           over all their entries; k and v written to their cache slot
//   pool_block_means        means of the cached keys / values of every block a row completes
//   unturn_gate             heads turned back by the row's position, times sigmoid(gate)
//   short_conv (+ tail)     causal per-channel filter over a step's rows and a sequence's kept inputs
//   rglru_scan              S <- d S + sqrt(1 - d^2) i u per channel, output S * gelu_tanh(y)
//   chosen_route            router logits + bias, top logits, softmax over the chosen, gate rows
//   capped_glu_route_scale  w * min(g, L) sigmoid(slope min(g, L)) (clamp(u, -L, L) + 1)
// Angles, gates, decays, state, router and every transcendental in fp32.
#include "hybrid_common.h"

using namespace hyb;

// ---------------------------------------------------------------------------------------
// One workgroup per token.  cos / sin of the row's angles once into LDS: cs[0 .. dims/2) cos,
// then sin, for q / k; the same for the values' E/2 angles behind them.  Caches contiguous
// [slot, G, D|E].  slot < 0: nothing is stored (q is still turned).
template <typename T>
__global__ void half_rope_store_kernel(T* __restrict__ q, const T* __restrict__ k,
                                       const T* __restrict__ v, long row_stride,
                                       const int* __restrict__ positions,
                                       const float* __restrict__ inv_freq, int dims,
                                       const float* __restrict__ v_inv_freq,
                                       T* __restrict__ k_cache, T* __restrict__ v_cache,
                                       const int* __restrict__ slot_mapping, int H, int G, int D, int E) {
    extern __shared__ float sm[];
    const long t = blockIdx.x;
    const int half = dims / 2, vhalf = v_inv_freq ? E / 2 : 0;
    float* cs = sm;                 // [2 * half]
    float* vcs = sm + 2 * half;     // [2 * vhalf]
    const float p = (float)positions[t];
    for (int i = threadIdx.x; i < half + vhalf; i += blockDim.x) {
        float s_, c_;
        if (i < half) {
            sincosf(p * inv_freq[i], &s_, &c_);
            cs[i] = c_; cs[half + i] = s_;
        } else {
            const int m = i - half;
            sincosf(p * v_inv_freq[m], &s_, &c_);
            vcs[m] = c_; vcs[vhalf + m] = s_;
        }
    }
    __syncthreads();
    T* qr = q + t * row_stride;
    for (int i = threadIdx.x; i < H * half; i += blockDim.x) {
        const int h = i / half, m = i - h * half;
        T* a = qr + (long)h * D + m;
        const float u = ld(a), w = ld(a + half), c = cs[m], s = cs[half + m];
        st(a, u * c - w * s);
        st(a + half, w * c + u * s);
    }
    const long slot = slot_mapping ? slot_mapping[t] : -1;
    if (slot < 0 || !k_cache) return;
    const T* kr = k + t * row_stride;
    for (int i = threadIdx.x; i < G * D; i += blockDim.x) {
        const int d = i % D;
        float o = ld(kr + i);
        if (d < half) o = o * cs[d] - ld(kr + i + half) * cs[half + d];
        else if (d < dims) o = o * cs[d - half] + ld(kr + i - half) * cs[d];
        st(k_cache + slot * (long)(G * D) + i, o);
    }
    const T* vr = v + t * row_stride;
    for (int i = threadIdx.x; i < G * E; i += blockDim.x) {
        const int e = i % E;
        float o = ld(vr + i);
        if (vhalf) {
            if (e < vhalf) o = o * vcs[e] - ld(vr + i + vhalf) * vcs[vhalf + e];
            else o = o * vcs[e - vhalf] + ld(vr + i - vhalf) * vcs[e];
        }
        st(v_cache + slot * (long)(G * E) + i, o);
    }
}

// Grid (row groups of POOL_ROWS rows, G), 256 threads.  A row whose position + 1 is a multiple of
// `pool` completes block blk = position / pool of its sequence: the fp32 sums of the block's
// cached rows, divided by pool, go to row (table[blk / prow] * prow + blk % prow) of the pooled
// caches.  A thread owns VEC consecutive columns of [key | value] and every `parts`-th cached row;
// the parts meet in LDS (parts * (D + E) floats).
constexpr int POOL_ROWS = 8;

template <typename T, int VEC>
__global__ void __launch_bounds__(256)
pool_block_means_kernel(const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                        T* __restrict__ k_pool, T* __restrict__ v_pool,
                        const int* __restrict__ positions, const int* __restrict__ slot_mapping,
                        const int* __restrict__ block_tables, int max_blocks,
                        const int* __restrict__ row_seq, long T_, int block_size, int pool,
                        int prow, int G, int D, int E, int parts) {
    extern __shared__ float red[];
    const int g = blockIdx.y, cols = D + E, cv = cols / VEC;
    const float inv = 1.f / (float)pool;
    for (int r = 0; r < POOL_ROWS; ++r) {
        const long t = (long)blockIdx.x * POOL_ROWS + r;
        if (t >= T_) break;
        const int p = positions[t];
        if (slot_mapping[t] < 0 || (p + 1) % pool) continue;            // (uniform)
        const int b = row_seq ? row_seq[t] : (int)t;
        if (b < 0) continue;
        const int* table = block_tables + (long)b * max_blocks;
        const int blk = p / pool, first = blk * pool;
        for (int idx = threadIdx.x; idx < parts * cv; idx += blockDim.x) {
            const int part = idx / cv, c = (idx - part * cv) * VEC;
            const bool isk = c < D;
            const T* src = isk ? k_cache + (long)g * D + c : v_cache + (long)g * E + (c - D);
            const long rs = isk ? (long)G * D : (long)G * E;
            float acc[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
#pragma unroll 8
            for (int j = first + part; j < first + pool; j += parts) {
                const long slot = (long)table[j / block_size] * block_size + j % block_size;
                float v[VEC];
                if constexpr (VEC == 1) v[0] = ld(src + slot * rs);
                else load_run<T, VEC>(src + slot * rs, v);
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc[i] += v[i];
            }
#pragma unroll
            for (int i = 0; i < VEC; ++i) red[part * cols + c + i] = acc[i];
        }
        __syncthreads();
        const long dst = (long)table[blk / prow] * prow + blk % prow;
        for (int c = threadIdx.x; c < cols; c += blockDim.x) {
            float sum = 0.f;
            for (int q = 0; q < parts; ++q) sum += red[q * cols + c];
            if (c < D) st(k_pool + (dst * G + g) * (long)D + c, sum * inv);
            else st(v_pool + (dst * G + g) * (long)E + (c - D), sum * inv);
        }
        __syncthreads();
    }
}

// out[t, h*E + m] = turned-back o[t, h, :] * sigmoid(gate[t, h*E + m]); o with strides (o_t, o_h, 1).
// vec: E/2 is a multiple of eight and every row 16-byte addressable - a thread then moves runs of
// eight columns of both halves of a head.
template <typename T>
__global__ void unturn_gate_kernel(const T* __restrict__ o, long o_t, long o_h,
                                   const int* __restrict__ positions,
                                   const float* __restrict__ v_inv_freq,
                                   const T* __restrict__ gate, long gate_stride,
                                   T* __restrict__ out, int H, int E, int vec) {
    extern __shared__ float sm[];
    const long t = blockIdx.x;
    const int half = E / 2;
    if (v_inv_freq) {
        const float p = (float)positions[t];
        for (int m = threadIdx.x; m < half; m += blockDim.x) {
            float s_, c_;
            sincosf(p * v_inv_freq[m], &s_, &c_);
            sm[m] = c_; sm[half + m] = s_;
        }
        __syncthreads();
    }
    const T* gr = gate ? gate + t * gate_stride : nullptr;
    T* orow = out + t * (long)(H * E);
    if (v_inv_freq && vec) {
        const int runs = half / 8;
        for (int i = threadIdx.x; i < H * runs; i += blockDim.x) {
            const int h = i / runs, m = (i - h * runs) * 8;
            const T* a = o + t * o_t + (long)h * o_h + m;
            float u[8], w[8], gu[8], gw[8], x[8], y[8];
            load_run<T, 8>(a, u);
            load_run<T, 8>(a + half, w);
            const int col = h * E + m;
            if (gr) { load_run<T, 8>(gr + col, gu); load_run<T, 8>(gr + col + half, gw); }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float c = sm[m + j], s = sm[half + m + j];
                x[j] = u[j] * c + w[j] * s;
                y[j] = w[j] * c - u[j] * s;
                if (gr) { x[j] *= sigmoidf_(gu[j]); y[j] *= sigmoidf_(gw[j]); }
            }
            store_run8<T>(orow + col, x);
            store_run8<T>(orow + col + half, y);
        }
    } else if (v_inv_freq) {
        for (int i = threadIdx.x; i < H * half; i += blockDim.x) {
            const int h = i / half, m = i - h * half;
            const T* a = o + t * o_t + (long)h * o_h + m;
            const float u = ld(a), w = ld(a + half), c = sm[m], s = sm[half + m];
            float x = u * c + w * s, y = w * c - u * s;          // the turn by minus the angle
            const int col = h * E + m;
            if (gr) { x *= sigmoidf_(ld(gr + col)); y *= sigmoidf_(ld(gr + col + half)); }
            st(orow + col, x);
            st(orow + col + half, y);
        }
    } else {
        for (int i = threadIdx.x; i < H * E; i += blockDim.x) {
            const int h = i / E, e = i - h * E;
            float x = ld(o + t * o_t + (long)h * o_h + e);
            if (gr) x *= sigmoidf_(ld(gr + i));
            st(orow + i, x);
        }
    }
}

// ---------------------------------------------------------------------------------------
// u[t, c] = bias[c] + sum_k w[c, k] x(t - (taps-1-k), c); grid (groups of CONV_ROWS rows, channel
// chunks); a thread owns VEC consecutive channels, keeps their taps (up to CONV_TAPS; longer filters
// read them from memory) in registers and walks the group's `rows_per` rows (CONV_ROWS for prompt
// portions, one for a handful of single tokens).  Inputs before the step's first
// row of the sequence come from tail [slots, taps-1, C] (the newest last); positions before the
// sequence's start count as zeros.  Rows of no sequence give zeros.
constexpr int CONV_ROWS = 8, CONV_TAPS = 8;

template <typename T, int VEC>
__global__ void short_conv_kernel(const T* __restrict__ x, long x_stride, const float* __restrict__ w,
                                  const float* __restrict__ bias, const float* __restrict__ tail,
                                  const int* __restrict__ cu_q, const int* __restrict__ positions,
                                  const int* __restrict__ slots, const int* __restrict__ row_seq,
                                  float* __restrict__ u, long T_, int C, int taps, int rows_per) {
    const int c = (blockIdx.y * blockDim.x + threadIdx.x) * VEC;
    if (c >= C) return;
    float wr[VEC][CONV_TAPS], b0[VEC];
    const bool inreg = taps <= CONV_TAPS;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        b0[i] = bias ? bias[c + i] : 0.f;
#pragma unroll
        for (int k = 0; k < CONV_TAPS; ++k) wr[i][k] = (inreg && k < taps) ? w[(long)(c + i) * taps + k] : 0.f;
    }
    for (int r = 0; r < rows_per; ++r) {
        const long t = (long)blockIdx.x * rows_per + r;
        if (t >= T_) return;
        const int b = cu_q ? row_seq[t] : (int)t;
        const int slot = b >= 0 ? slots[b] : -1;
        float acc[VEC];
        if (slot < 0) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) u[t * C + c + i] = 0.f;
            continue;
        }
        const long s0 = cu_q ? cu_q[b] : t;
        const int off = (int)(t - s0), pos = positions[t];
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = b0[i];
        auto input = [&](int d, float* xv) {
            if (off - d >= 0) {
                if constexpr (VEC == 1) xv[0] = ld(x + (t - d) * x_stride + c);
                else load_run<T, VEC>(x + (t - d) * x_stride + c, xv);
            } else {
                const float* tp = tail + ((long)slot * (taps - 1) + (taps - 1 + off - d)) * C + c;
#pragma unroll
                for (int i = 0; i < VEC; ++i) xv[i] = tp[i];
            }
        };
        if (inreg) {
#pragma unroll
            for (int k = 0; k < CONV_TAPS; ++k) {
                const int d = taps - 1 - k;
                if (k < taps && pos - d >= 0) {
                    float xv[VEC];
                    input(d, xv);
#pragma unroll
                    for (int i = 0; i < VEC; ++i) acc[i] += wr[i][k] * xv[i];
                }
            }
        } else {
            for (int k = 0; k < taps; ++k) {
                const int d = taps - 1 - k;
                if (pos - d < 0) continue;
                float xv[VEC];
                input(d, xv);
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc[i] += w[(long)(c + i) * taps + k] * xv[i];
            }
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) u[t * C + c + i] = acc[i];
    }
}

// The kept inputs after the step: grid (channel chunks, sequences); runs after every row has read.
template <typename T>
__global__ void short_conv_tail_kernel(const T* __restrict__ x, long x_stride, float* __restrict__ tail,
                                       const int* __restrict__ cu_q, const int* __restrict__ positions,
                                       const int* __restrict__ slots, int C, int taps) {
    const int b = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int slot = slots[b];
    if (slot < 0) return;
    const long s0 = cu_q ? cu_q[b] : b, e0 = cu_q ? cu_q[b + 1] : b + 1;
    const int n = (int)(e0 - s0);
    if (n <= 0) return;
    const int p0 = positions[s0], keep = taps - 1;
    float* tl = tail + (long)slot * keep * C + c;
    for (int i = 0; i < keep; ++i) {                  // ascending: reads never trail the writes
        const int off = n - keep + i;                 // row offset inside the step
        float v;
        if (off >= 0) v = ld(x + (s0 + off) * x_stride + c);
        else v = (p0 + off >= 0) ? tl[(long)(i + n) * C] : 0.f;
        tl[(long)i * C] = v;
    }
}

// sigmoid on the hardware exponential and reciprocal (both within a few ulp): the scan evaluates
// three per element and pass
__device__ __forceinline__ float fast_sigmoid(float z) { return __fdividef(1.f, 1.f + __expf(-z)); }

// 0.5 z (1 + tanh(a)) = z sigmoid(2 a), a = sqrt(2/pi) (z + 0.044715 z^3)
__device__ __forceinline__ float gelu_tanh_(float z) {
    return z * fast_sigmoid(1.5957691216057308f * (z + 0.044715f * z * z * z));
}

// 1 - exp(t) for t <= 0 without cancellation: the series next to zero, 1 - exp(t) elsewhere
__device__ __forceinline__ float one_minus_exp(float t, float e) {
    const float series = -t * (1.f + t * (0.5f + t * (1.f / 6.f + t * (1.f / 24.f + t * (1.f / 120.f +
                               t * (1.f / 720.f + t * (1.f / 5040.f)))))));
    return t > -0.25f ? series : 1.f - e;
}

// Workgroup = 64 channels x nw waves of one sequence; wave w walks the w-th part of the
// sequence's rows.  With nw > 1 a first pass folds each part into (A, B) with S_end = A S_in + B,
// the parts' carries meet in LDS, and a second pass walks the part again from its true S_in and
// writes the outputs.  gates [nb, T, 2c]: for channel k c + j the recurrence gate's
// pre-activation at [k, t, j], the input gate's at [k, t, c + j].
struct GateStep { float d, add; };

__device__ __forceinline__ GateStep rglru_step(const float* __restrict__ gates, const float* __restrict__ u,
                                               long t, long T_, int C, int c2, long gcol, int ch,
                                               float br, float bi, float nsp) {
    const float* gp = gates + t * c2 + gcol;
    const float r = fast_sigmoid(gp[0] + br), i = fast_sigmoid(gp[c2 / 2] + bi);
    const float la = nsp * r;                                   // log of the decay
    GateStep s;
    s.d = __expf(la);
    s.add = sqrtf(one_minus_exp(2.f * la, s.d * s.d)) * i * u[t * C + ch];      // sqrt(1 - d^2)
    return s;
}

template <typename T>
__global__ void rglru_scan_kernel(const float* __restrict__ u, const float* __restrict__ gates,
                                  const float* __restrict__ gate_bias, const float* __restrict__ lam,
                                  const T* __restrict__ y, long y_stride, float* __restrict__ state,
                                  const int* __restrict__ cu_q, const int* __restrict__ positions,
                                  const int* __restrict__ slots, T* __restrict__ out, long T_,
                                  int C, int nb, float sharp) {
    extern __shared__ float sm[];                    // [nw][64][2]
    const int b = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int slot = slots[b];
    const long s0 = cu_q ? cu_q[b] : b, e0 = cu_q ? cu_q[b + 1] : b + 1;
    if (slot < 0 || e0 <= s0) return;                // the whole workgroup leaves
    const int chr = blockIdx.x * 64 + lane;
    const bool live = chr < C;
    const int ch = live ? chr : C - 1;
    const int c = C / nb, k = ch / c, j = ch - k * c, c2 = 2 * c;
    const long gcol = (long)k * T_ * c2 + j;
    const float br = gate_bias[k * c2 + j], bi = gate_bias[k * c2 + c + j];
    const float nsp = -sharp * softplusf_(lam[ch]);
    const long n = e0 - s0, part = (n + nw - 1) / nw;
    const long lo = s0 + wave * part, hi = lo + part < e0 ? lo + part : e0;
    float S = positions[s0] > 0 ? state[(long)slot * C + ch] : 0.f;
    if (nw > 1) {
        float A = 1.f, B = 0.f;
        for (long t = lo; t < hi; ++t) {
            const GateStep g = rglru_step(gates, u, t, T_, C, c2, gcol, ch, br, bi, nsp);
            A *= g.d;
            B = g.d * B + g.add;
        }
        sm[(wave * 64 + lane) * 2] = A;
        sm[(wave * 64 + lane) * 2 + 1] = B;
        __syncthreads();
        for (int v = 0; v < wave; ++v) S = sm[(v * 64 + lane) * 2] * S + sm[(v * 64 + lane) * 2 + 1];
    }
    for (long t = lo; t < hi; ++t) {
        const GateStep g = rglru_step(gates, u, t, T_, C, c2, gcol, ch, br, bi, nsp);
        S = g.d * S + g.add;
        if (live) st(out + t * C + ch, S * gelu_tanh_(ld(y + t * y_stride + ch)));
    }
    if (wave == nw - 1 && live) state[(long)slot * C + ch] = S;
}

// ---------------------------------------------------------------------------------------
// One workgroup (256 threads) per token: fp32 logits of NR = NE + gates rows of wr (+ bias), the
// `top` largest of the first NE chosen (ties to the lower index), dense[t, e] = softmax over the
// chosen logits, zero elsewhere; dense[t, NE + i] = sigmoid(logit of gate row i).  LDS: NR + 32.
template <typename T>
__global__ void chosen_route_kernel(const T* __restrict__ h, const float* __restrict__ wr,
                                    const float* __restrict__ bias, float* __restrict__ dense,
                                    int W, int NE, int NR, int top) {
    extern __shared__ float sm[];
    float* z = sm;
    float* red = sm + NR;       // [4 waves][8]
    const long t = blockIdx.x;
    const T* hr = h + t * W;
    for (int e0 = 0; e0 < NR; e0 += 8) {
        float acc[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = 0.f;
#pragma unroll 4
        for (int c = threadIdx.x; c < W; c += blockDim.x) {
            const float hv = ld(hr + c);
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (e0 + j < NR) acc[j] += hv * wr[(long)(e0 + j) * W + c];
        }
        const int wave = threadIdx.x / kWave, nw = blockDim.x / kWave;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float sj = wave_sum(acc[j]);
            if ((threadIdx.x & (kWave - 1)) == 0) red[wave * 8 + j] = sj;
        }
        __syncthreads();
        if (threadIdx.x < 8 && e0 + threadIdx.x < NR) {
            float sj = bias ? bias[e0 + threadIdx.x] : 0.f;
            for (int w = 0; w < nw; ++w) sj += red[w * 8 + threadIdx.x];
            z[e0 + threadIdx.x] = sj;
        }
        __syncthreads();
    }
    float* row = dense + t * NR;
    for (int e = threadIdx.x; e < NR; e += blockDim.x) row[e] = e < NE ? 0.f : sigmoidf_(z[e]);
    __syncthreads();
    if (threadIdx.x == 0) {
        float best = 0.f, sum = 0.f;
        for (int r = 0; r < top; ++r) {              // the r-th largest logit not yet taken
            int be = -1; float bv = -INFINITY;
            for (int e = 0; e < NE; ++e) if (z[e] > bv) { bv = z[e]; be = e; }
            if (be < 0) break;                       // (logits that are not numbers)
            if (r == 0) best = bv;
            const float p = expf(bv - best);
            row[be] = p;
            sum += p;
            z[be] = -INFINITY;                       // taken
        }
        const float inv = 1.f / sum;
        for (int e = 0; e < NE; ++e) row[e] *= inv;
    }
}

// gu row = [gate columns C | up columns C], C = NE * ff + sff; dense [T, NR], NR = NE (+ 1: the
// shared columns' gate).  VEC consecutive columns per thread (VEC divides ff, sff, the strides).
template <typename T, int VEC>
__global__ void capped_glu_route_scale_kernel(const T* __restrict__ gu, long gu_stride,
                                              const float* __restrict__ dense, T* __restrict__ act,
                                              int NE, int NR, int ff, int C, float limit,
                                              float shared_limit, float slope) {
    const long t = blockIdx.y;
    const T* g = gu + t * gu_stride;
    const T* u = g + C;
    const int routed = NE * ff;
    for (int c = (blockIdx.x * blockDim.x + threadIdx.x) * VEC; c < C; c += gridDim.x * blockDim.x * VEC) {
        const bool sh = c >= routed;
        const float w = sh ? (NR > NE ? dense[t * NR + NE] : 1.f) : dense[t * NR + c / ff];
        const float L = sh ? shared_limit : limit;
        float gv[VEC], uv[VEC];
        if (w != 0.f) {
            if constexpr (VEC == 1) { gv[0] = ld(g + c); uv[0] = ld(u + c); }
            else { load_run<T, VEC>(g + c, gv); load_run<T, VEC>(u + c, uv); }
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float gg = fminf(gv[j], L), uu = fminf(fmaxf(uv[j], -L), L);
                gv[j] = w * (gg * sigmoidf_(slope * gg) * (uu + 1.f));
            }
        } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) gv[j] = 0.f;
        }
#pragma unroll
        for (int j = 0; j < VEC; ++j) st(act + t * (long)C + c + j, gv[j]);
    }
}

static inline int threads_for(int n) { return n >= 1024 ? 512 : n >= 256 ? 256 : n > 64 ? 128 : 64; }

extern "C" {

int hyb_half_rope_store(void* q, const void* k, const void* v, long row_stride, const void* positions,
                        const void* inv_freq, int dims, const void* v_inv_freq, void* k_cache,
                        void* v_cache, const void* slot_mapping, long T_, int H, int G, int D, int E,
                        int dt, hipStream_t s) {
    if (T_ <= 0) return 0;
    if (dims < 0 || dims % 2 || dims > D || (v_inv_freq && E % 2) || (dims && !inv_freq)) return 1;
    const size_t lds = (dims + (v_inv_freq ? E : 0) + 1) * sizeof(float);
    HYB_DISPATCH(dt, hipLaunchKernelGGL(half_rope_store_kernel<T>, dim3(T_), dim3(threads_for(H * D / 2)),
                                        lds, s, (T*)q, (const T*)k, (const T*)v, row_stride,
                                        (const int*)positions, (const float*)inv_freq, dims,
                                        (const float*)v_inv_freq, (T*)k_cache, (T*)v_cache,
                                        (const int*)slot_mapping, H, G, D, E));
    return HYB_LAUNCH_OK();
}

int hyb_pool_block_means(const void* k_cache, const void* v_cache, void* k_pool, void* v_pool,
                         const void* positions, const void* slot_mapping, const void* block_tables,
                         int max_blocks, const void* row_seq, long T_, int block_size, int pool,
                         int prow, int G, int D, int E, int dt, hipStream_t s) {
    if (T_ <= 0) return 0;
    if (pool <= 0 || prow <= 0 || (long)prow * pool < block_size || !slot_mapping) return 1;
    const bool vec = D % 4 == 0 && E % 4 == 0 && (size_t)k_cache % 16 == 0 && (size_t)v_cache % 16 == 0;
    const int cv = (D + E) / (vec ? 4 : 1);
    int parts = 256 / cv;
    parts = parts < 1 ? 1 : (parts > pool ? pool : parts);
    const dim3 grid((unsigned)((T_ + POOL_ROWS - 1) / POOL_ROWS), G);
    const size_t lds = (size_t)parts * (D + E) * sizeof(float);
#define POOL_LAUNCH(VEC)                                                                          \
    HYB_DISPATCH(dt, hipLaunchKernelGGL((pool_block_means_kernel<T, VEC>), grid, dim3(256), lds, s, \
                                        (const T*)k_cache, (const T*)v_cache, (T*)k_pool,         \
                                        (T*)v_pool, (const int*)positions,                        \
                                        (const int*)slot_mapping, (const int*)block_tables,       \
                                        max_blocks, (const int*)row_seq, T_, block_size, pool,    \
                                        prow, G, D, E, parts))
    if (vec) POOL_LAUNCH(4); else POOL_LAUNCH(1);
#undef POOL_LAUNCH
    return HYB_LAUNCH_OK();
}

int hyb_unturn_gate(const void* o, long o_t, long o_h, const void* positions, const void* v_inv_freq,
                    const void* gate, long gate_stride, void* out, long T_, int H, int E, int dt,
                    hipStream_t s) {
    if (T_ <= 0) return 0;
    if (v_inv_freq && E % 2) return 1;
    const int vec = v_inv_freq && E % 16 == 0 && o_t % 8 == 0 && o_h % 8 == 0 && gate_stride % 8 == 0 &&
                    ((size_t)o | (size_t)gate | (size_t)out) % 16 == 0;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(unturn_gate_kernel<T>, dim3(T_),
                                        dim3(threads_for(vec ? H * E / 16 : H * E / 2)),
                                        (E + 1) * sizeof(float), s, (const T*)o, o_t, o_h,
                                        (const int*)positions, (const float*)v_inv_freq,
                                        (const T*)gate, gate_stride, (T*)out, H, E, vec));
    return HYB_LAUNCH_OK();
}

// x [T, C] rows x_stride apart; u [T, C] fp32; tail [slots, taps-1, C] fp32 (updated); B sequences
int hyb_short_conv(const void* x, long x_stride, const void* w, const void* bias, void* tail,
                   const void* cu_q, const void* positions, const void* slots, const void* row_seq,
                   void* u, long T_, int B, int C, int taps, int dt, hipStream_t s) {
    if (T_ <= 0 || C <= 0) return 0;
    if (taps < 1 || (cu_q && !row_seq) || (taps > 1 && !tail) || B > 65535) return 1;
    const int esize = dt == 0 ? 2 : 4;
    const bool vec = C % 4 == 0 && x_stride % 4 == 0 && (size_t)x % (4 * esize) == 0;
    const int th = threads_for(C), bx = (C + th - 1) / th;
    const int thv = threads_for(C / 4), bxv = (C / 4 + thv - 1) / thv;
    const int rows_per = T_ >= 2048 ? CONV_ROWS : 1;
#define CONV_LAUNCH(VEC, nb_, nt_)                                                                \
    HYB_DISPATCH(dt, hipLaunchKernelGGL((short_conv_kernel<T, VEC>),                              \
                                        dim3((unsigned)((T_ + rows_per - 1) / rows_per), nb_),    \
                                        dim3(nt_), 0, s,                                          \
                                        (const T*)x, x_stride, (const float*)w, (const float*)bias, \
                                        (const float*)tail, (const int*)cu_q, (const int*)positions, \
                                        (const int*)slots, (const int*)row_seq, (float*)u, T_, C, taps, \
                                        rows_per))
    if (vec) CONV_LAUNCH(4, bxv, thv); else CONV_LAUNCH(1, bx, th);
#undef CONV_LAUNCH
    if (hipGetLastError() != hipSuccess) return 2;
    if (taps > 1 && B > 0)
        HYB_DISPATCH(dt, hipLaunchKernelGGL(short_conv_tail_kernel<T>, dim3(bx, B), dim3(th), 0, s,
                                            (const T*)x, x_stride, (float*)tail, (const int*)cu_q,
                                            (const int*)positions, (const int*)slots, C, taps));
    return HYB_LAUNCH_OK();
}

// nw: waves (parts of a sequence's rows) per workgroup, 1 .. 16
int hyb_rglru_scan(const void* u, const void* gates, const void* gate_bias, const void* lam,
                   const void* y, long y_stride, void* state, const void* cu_q, const void* positions,
                   const void* slots, void* out, long T_, int B, int C, int nb, float sharp, int nw,
                   int dt, hipStream_t s) {
    if (T_ <= 0 || B <= 0) return 0;
    if (nb < 1 || C % nb || nw < 1 || nw > 16 || B > 65535) return 1;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(rglru_scan_kernel<T>, dim3((C + 63) / 64, B), dim3(64 * nw),
                                        nw * 64 * 2 * sizeof(float), s, (const float*)u,
                                        (const float*)gates, (const float*)gate_bias, (const float*)lam,
                                        (const T*)y, y_stride, (float*)state, (const int*)cu_q,
                                        (const int*)positions, (const int*)slots, (T*)out, T_, C, nb,
                                        sharp));
    return HYB_LAUNCH_OK();
}

int hyb_chosen_route(const void* h, const void* wr, const void* bias, void* dense, long T_, int W,
                     int NE, int NR, int top, int dt, hipStream_t s) {
    if (T_ <= 0) return 0;
    if (NE < 1 || NR < NE || top < 1 || top > NE || NR > 4096) return 1;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(chosen_route_kernel<T>, dim3(T_), dim3(256),
                                        (NR + 32) * sizeof(float), s, (const T*)h, (const float*)wr,
                                        (const float*)bias, (float*)dense, W, NE, NR, top));
    return HYB_LAUNCH_OK();
}

int hyb_capped_glu_route_scale(const void* gu, long gu_stride, const void* dense, void* act, long T_,
                               int NE, int NR, int ff, int sff, float limit, float shared_limit,
                               float slope, int dt, hipStream_t s) {
    const int C = NE * ff + sff;
    if (T_ <= 0 || C <= 0) return 0;
    if (!dense || NR < NE) return 1;
    const int esize = dt == 0 ? 2 : 4;
    const bool vec = (NE == 0 || ff % 8 == 0) && sff % 8 == 0 && gu_stride % 8 == 0 &&
                     (size_t)gu % (4 * esize) == 0 && (C * (size_t)esize) % (4 * esize) == 0;
    const int per = vec ? 8 : 1;
    const int need = (C / per + 255) / 256;
    const int bx = need > 64 ? 64 : (need < 1 ? 1 : need);
    for (long t0 = 0; t0 < T_; t0 += 65535) {          // blockIdx.y holds at most 65535 rows
        const long n = T_ - t0 < 65535 ? T_ - t0 : 65535;
#define CGLU(VEC)                                                                                 \
        HYB_DISPATCH(dt, hipLaunchKernelGGL((capped_glu_route_scale_kernel<T, VEC>), dim3(bx, n),  \
                                            dim3(256), 0, s, (const T*)gu + t0 * gu_stride,       \
                                            gu_stride, (const float*)dense + t0 * NR,             \
                                            (T*)act + t0 * (long)C, NE, NR, ff, C, limit,         \
                                            shared_limit, slope))
        if (vec) CGLU(8); else CGLU(1);
#undef CGLU
    }
    return HYB_LAUNCH_OK();
}

}  // extern "C"
