// Row-wise kernels of hybrid decoders: embedding sum, zero-centred RMS norms around a fp32
// residual stream, rotation of neighbouring pairs + value mixing + KV store, gated per-head
// norm, grouped expert routing and the routed gelu.  One workgroup per token row unless noted.
#include "hybrid_common.h"

using namespace hyb;

// x[t] = (table[ids[t]] + aux[aux_rows[t]]) * scale  (fp32 out)
template <typename T>
__global__ void embed_sum_kernel(const int* __restrict__ ids, const int* __restrict__ aux_rows,
                                 const T* __restrict__ table, const T* __restrict__ aux,
                                 float* __restrict__ x, int W, float scale) {
    const long t = blockIdx.x;
    const T* a = table + (long)ids[t] * W;
    const T* b = aux ? aux + (long)aux_rows[t] * W : nullptr;
    for (int c = threadIdx.x; c < W; c += blockDim.x)
        x[t * W + c] = (ld(a + c) + (b ? ld(b + c) : 0.f)) * scale;
}

// out[t] = x[t] / rms(x[t]) * (1 + w)
template <typename T>
__global__ void offset_rms_norm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                       T* __restrict__ out, int W, float eps) {
    __shared__ float red[16];
    const long t = blockIdx.x;
    const float* xr = x + t * W;
    float s = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) { const float v = xr[c]; s += v * v; }
    const float r = rsqrtf(block_sum(s, red) / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x) st(out + t * W + c, xr[c] * r * (1.f + w[c]));
}

// x[t] += y[t] / rms(y[t]) * (1 + wb);  h[t] = x[t] / rms(x[t]) * (1 + wn)   (h optional)
template <typename T>
__global__ void post_norm_residual_kernel(const T* __restrict__ y, long y_stride,
                                          const float* __restrict__ wb, float* __restrict__ x,
                                          const float* __restrict__ wn, T* __restrict__ h, int W,
                                          float eps) {
    __shared__ float red[16];
    const long t = blockIdx.x;
    const T* yr = y + t * y_stride;
    float* xr = x + t * W;
    float s = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) { const float v = ld(yr + c); s += v * v; }
    const float r = rsqrtf(block_sum(s, red) / (float)W + eps);
    float s2 = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float v = xr[c] + ld(yr + c) * r * (1.f + wb[c]);
        xr[c] = v;
        s2 += v * v;
    }
    if (!h) return;
    const float r2 = rsqrtf(block_sum(s2, red) / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x) st(h + t * W + c, xr[c] * r2 * (1.f + wn[c]));
}

// Per token: rotate q in place (pairs (2i, 2i+1) of the first rot entries of each head), rotate k
// and write it to its cache slot, write v (optionally published to / blended with v_first) to
// its slot.  cos_sin [max_pos, rot]: cos then sin.  Caches are contiguous [slot, G, D|E].
template <typename T>
__global__ void pair_rope_mix_store_kernel(T* __restrict__ q, const T* __restrict__ k,
                                           const T* __restrict__ v, long row_stride,
                                           const int* __restrict__ positions,
                                           const float* __restrict__ cos_sin, int rot,
                                           T* __restrict__ v_first, const float* __restrict__ lam,
                                           int v_mode, T* __restrict__ k_cache,
                                           T* __restrict__ v_cache,
                                           const int* __restrict__ slot_mapping, int H, int G,
                                           int D, int E) {
    const long t = blockIdx.x;
    const int p = positions[t];
    const long slot = slot_mapping ? slot_mapping[t] : -1;
    const float* cs = cos_sin ? cos_sin + (long)p * rot : nullptr;
    const int half = rot / 2;
    T* qr = q + t * row_stride;
    for (int i = threadIdx.x; i < H * half; i += blockDim.x) {
        const int hh = i / half, j = i - hh * half;
        T* a = qr + hh * D + 2 * j;
        const float c = cs[j], s = cs[half + j], u = ld(a), w = ld(a + 1);
        st(a, u * c - w * s);
        st(a + 1, w * c + u * s);
    }
    const T* kr = k + t * row_stride;
    if (slot >= 0 && k_cache) {
        T* kc = k_cache + slot * (long)(G * D);
        for (int i = threadIdx.x; i < G * D; i += blockDim.x) {
            const int d = i % D;
            float val;
            if (d < rot) {
                const int j = d >> 1;
                const float c = cs[j], s = cs[half + j];
                const int base = i - d;
                const float u = ld(kr + base + (d & ~1)), w = ld(kr + base + (d | 1));
                val = (d & 1) ? (w * c + u * s) : (u * c - w * s);
            } else {
                val = ld(kr + i);
            }
            st(kc + i, val);
        }
    }
    const T* vr = v + t * row_stride;
    const float l = (v_mode == 2) ? *lam : 0.f;
    for (int i = threadIdx.x; i < G * E; i += blockDim.x) {
        float val = ld(vr + i);
        if (v_mode == 1) st(v_first + t * (long)(G * E) + i, val);
        if (v_mode == 2) val = (1.f - l) * val + l * ld(v_first + t * (long)(G * E) + i);
        if (slot >= 0 && v_cache) st(v_cache + slot * (long)(G * E) + i, val);
    }
}

// out[t,h,:] = o[t,h,:] / rms(o[t,h,:]) * w * act(gate[t,h,:]); one wave per (t, h).  w_heads: w
// has H * E entries (0: E entries shared by the heads); sig: act is the sigmoid (0: silu).
template <typename T>
__global__ void gated_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                       const T* __restrict__ gate, long gate_stride,
                                       T* __restrict__ out, int H, int E, float eps, int w_heads,
                                       int sig) {
    const long th = blockIdx.x;
    const long t = th / H;
    const int h = th - t * H;
    const float* orow = o + th * E;
    float s = 0.f;
    for (int e = threadIdx.x; e < E; e += kWave) { const float v = orow[e]; s += v * v; }
    const float r = rsqrtf(wave_sum(s) / (float)E + eps);
    const T* g = gate + t * gate_stride + (long)h * E;
    const float* wh = w + (w_heads ? (long)h * E : 0);
    for (int e = threadIdx.x; e < E; e += kWave) {
        const float z = ld(g + e);
        st(out + th * E + e, orow[e] * r * wh[e] * (sig ? sigmoidf_(z) : siluf_(z)));
    }
}

// One workgroup (256 threads) per token: fp32 router logits (the row is read once, eight experts'
// partial sums per pass), softmax over all experts (sig: the sigmoid of each logit instead), best
// `keep` of `groups` groups (a group scores its best expert), `top` largest eligible scores; dense
// [T, NE] out, zero where not chosen.  Ties go to the lower index.  LDS: 2 * NE + 32 floats.
template <typename T>
__global__ void grouped_route_kernel(const T* __restrict__ h, const float* __restrict__ wr,
                                     float* __restrict__ dense, int W, int NE, int top,
                                     int groups, int keep, int sig) {
    extern __shared__ float sm[];
    float* z = sm;              // scores
    float* elig = sm + NE;      // eligible scores (or -1)
    float* red = sm + 2 * NE;   // [4 waves][8]
    const long t = blockIdx.x;
    const T* hr = h + t * W;
    for (int e0 = 0; e0 < NE; e0 += 8) {
        float acc[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = 0.f;
#pragma unroll 4
        for (int c = threadIdx.x; c < W; c += blockDim.x) {
            const float hv = ld(hr + c);
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (e0 + j < NE) acc[j] += hv * wr[(long)(e0 + j) * W + c];
        }
        // eight sums at once: per wave by exchanges, across the 4 waves through LDS
        const int wave = threadIdx.x / kWave, nw = blockDim.x / kWave;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float sj = wave_sum(acc[j]);
            if ((threadIdx.x & (kWave - 1)) == 0) red[wave * 8 + j] = sj;
        }
        __syncthreads();
        if (threadIdx.x < 8 && e0 + threadIdx.x < NE) {
            float sj = 0.f;
            for (int w = 0; w < nw; ++w) sj += red[w * 8 + threadIdx.x];
            z[e0 + threadIdx.x] = sj;
        }
        __syncthreads();
    }
    if (threadIdx.x < kWave && sig) {            // every expert scored by the sigmoid of its own logit
        for (int e = threadIdx.x; e < NE; e += kWave) {
            z[e] = sigmoidf_(z[e]);
            elig[e] = -1.f;
            dense[t * NE + e] = 0.f;
        }
    } else if (threadIdx.x < kWave) {
        float m = -INFINITY;
        for (int e = threadIdx.x; e < NE; e += kWave) m = fmaxf(m, z[e]);
        m = wave_max(m);
        float sum = 0.f;
        for (int e = threadIdx.x; e < NE; e += kWave) sum += expf(z[e] - m);
        sum = wave_sum(sum);
        for (int e = threadIdx.x; e < NE; e += kWave) {
            z[e] = expf(z[e] - m) / sum;
            elig[e] = -1.f;
            dense[t * NE + e] = 0.f;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int per = NE / groups;
        // mark the kept groups: repeatedly take the best unmarked group
        for (int r = 0; r < keep; ++r) {
            int bg = -1; float bv = -1.f;
            for (int g = 0; g < groups; ++g) {
                if (elig[g * per] >= 0.f) continue;          // already kept
                float gv = z[g * per];
                for (int j = 1; j < per; ++j) gv = fmaxf(gv, z[g * per + j]);
                if (gv > bv) { bv = gv; bg = g; }
            }
            for (int j = 0; j < per; ++j) elig[bg * per + j] = z[bg * per + j];
        }
        for (int r = 0; r < top; ++r) {
            int be = -1; float bv = -1.f;
            for (int e = 0; e < NE; ++e) if (elig[e] > bv) { bv = elig[e]; be = e; }
            dense[t * NE + be] = z[be];
            elig[be] = -2.f;
        }
    }
}

// act[t, e*ff + j] = gelu(up[t, e*ff + j]) * dense[t, e]; VEC elements per thread and step (one
// expert lookup per run; ff % VEC == 0)
template <typename T, int VEC>
__global__ void gelu_route_scale_kernel(const T* __restrict__ up, const float* __restrict__ dense,
                                        T* __restrict__ act, long n, int NE, int ff) {
    const long cols = (long)NE * ff;
    for (long i = (blockIdx.x * (long)blockDim.x + threadIdx.x) * VEC; i < n;
         i += (long)gridDim.x * blockDim.x * VEC) {
        const long t = i / cols;
        const int e = (int)((i - t * cols) / ff);
        const float w = dense[t * NE + e];
        if (w == 0.f) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) st(act + i + j, 0.f);
        } else {
            float v[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] = ld(up + i + j);
#pragma unroll
            for (int j = 0; j < VEC; ++j) st(act + i + j, gelu_erf(v[j]) * w);
        }
    }
}

static inline int threads_for(int n) { return n >= 1024 ? 512 : n >= 256 ? 256 : n > 64 ? 128 : 64; }

extern "C" {

int hyb_embed_sum(const void* ids, const void* aux_rows, const void* table, const void* aux,
                  void* x, long T_, int W, float scale, int dt, hipStream_t s) {
    if (T_ <= 0) return 0;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(embed_sum_kernel<T>, dim3(T_), dim3(threads_for(W)), 0, s,
                                        (const int*)ids, (const int*)aux_rows, (const T*)table,
                                        (const T*)aux, (float*)x, W, scale));
    return HYB_LAUNCH_OK();
}

int hyb_offset_rms_norm(const void* x, const void* w, void* out, long T_, int W, float eps, int dt,
                        hipStream_t s) {
    if (T_ <= 0) return 0;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(offset_rms_norm_kernel<T>, dim3(T_), dim3(threads_for(W)),
                                        0, s, (const float*)x, (const float*)w, (T*)out, W, eps));
    return HYB_LAUNCH_OK();
}

int hyb_post_norm_residual(const void* y, long y_stride, const void* wb, void* x, const void* wn,
                           void* h, long T_, int W, float eps, int dt, hipStream_t s) {
    if (T_ <= 0) return 0;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(post_norm_residual_kernel<T>, dim3(T_),
                                        dim3(threads_for(W)), 0, s, (const T*)y, y_stride,
                                        (const float*)wb, (float*)x, (const float*)wn, (T*)h, W, eps));
    return HYB_LAUNCH_OK();
}

int hyb_pair_rope_mix_store(void* q, const void* k, const void* v, long row_stride,
                            const void* positions, const void* cos_sin, int rot, void* v_first,
                            const void* lam, int v_mode, void* k_cache, void* v_cache,
                            const void* slot_mapping, long T_, int H, int G, int D, int E, int dt,
                            hipStream_t s) {
    if (T_ <= 0) return 0;
    if (rot & 1 || rot > D || (rot > 0 && !cos_sin)) return 1;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(pair_rope_mix_store_kernel<T>, dim3(T_), dim3(256), 0, s,
                                        (T*)q, (const T*)k, (const T*)v, row_stride,
                                        (const int*)positions, (const float*)cos_sin, rot,
                                        (T*)v_first, (const float*)lam, v_mode, (T*)k_cache,
                                        (T*)v_cache, (const int*)slot_mapping, H, G, D, E));
    return HYB_LAUNCH_OK();
}

int hyb_gated_head_norm(const void* o, const void* w, const void* gate, long gate_stride,
                        void* out, long T_, int H, int E, float eps, int w_heads, int sig, int dt,
                        hipStream_t s) {
    if (T_ <= 0) return 0;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(gated_head_norm_kernel<T>, dim3(T_ * H), dim3(kWave), 0, s,
                                        (const float*)o, (const float*)w, (const T*)gate,
                                        gate_stride, (T*)out, H, E, eps, w_heads, sig));
    return HYB_LAUNCH_OK();
}

int hyb_grouped_route(const void* h, const void* wr, void* dense, long T_, int W, int NE, int top,
                      int groups, int keep, int sig, int dt, hipStream_t s) {
    if (T_ <= 0) return 0;
    if (groups <= 0 || NE % groups || keep > groups || top > NE / groups * keep || NE > 4096) return 1;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(grouped_route_kernel<T>, dim3(T_), dim3(256),
                                        (2 * NE + 32) * sizeof(float), s, (const T*)h, (const float*)wr,
                                        (float*)dense, W, NE, top, groups, keep, sig));
    return HYB_LAUNCH_OK();
}

int hyb_gelu_route_scale(const void* up, const void* dense, void* act, long T_, int NE, int ff,
                         int dt, hipStream_t s) {
    const long n = T_ * NE * ff;
    if (n <= 0) return 0;
    if (ff % 8 == 0) {
        const long work = n / 8;
        const int blocks = (int)((work + 255) / 256 > 16384 ? 16384 : (work + 255) / 256);
        HYB_DISPATCH(dt, hipLaunchKernelGGL((gelu_route_scale_kernel<T, 8>), dim3(blocks), dim3(256),
                                            0, s, (const T*)up, (const float*)dense, (T*)act, n, NE, ff));
    } else {
        const int blocks = (int)((n + 255) / 256 > 16384 ? 16384 : (n + 255) / 256);
        HYB_DISPATCH(dt, hipLaunchKernelGGL((gelu_route_scale_kernel<T, 1>), dim3(blocks), dim3(256),
                                            0, s, (const T*)up, (const float*)dense, (T*)act, n, NE, ff));
    }
    return HYB_LAUNCH_OK();
}

}  // extern "C"
