// Row-wise kernels of decoders whose parallel branches are added to a fp32 stream with a scale
// each and normed with a single gain, and of attention over a shared latent:
//   residual_sum_norm   x += sum_i s_i y_i;  h = x / rms(x) * gain       (the next layer's input)
//   rms_norm_rows       rows of an activation tensor / rms * w            (a latent's norm)
//   row_norm_store      q and k RMS-normed over their WHOLE projection (all heads at once), or
//                       left as they are; k and v written to their cache slot
//   latent_rope_store   latent norm + half-split rotation + query assembly + cache write
//   xielu               the piecewise quadratic / exponential activation
//   gated_group_norm    (o + skip x) silu(z), RMS norm in equal parts, weight
//   sigmoid_gate        o * sigmoid(g) element by element, gathering a head-major o
// One workgroup per token row unless noted; every reduction, angle and transcendental in fp32.
#include "hybrid_common.h"

using namespace hyb;

constexpr int MAX_BRANCHES = 4;

struct Branches {
    const void* y[MAX_BRANCHES];
    long stride[MAX_BRANCHES];
    float scale[MAX_BRANCHES];
    int n;
};

// x [T, W] fp32 updated in place; h [T, W] (or null) = x / sqrt(mean(x^2) + eps) * gain.
template <typename T>
__global__ void residual_sum_norm_kernel(float* __restrict__ x, Branches br, float gain,
                                         T* __restrict__ h, int W, float eps) {
    __shared__ float red[16];
    const long t = blockIdx.x;
    float* xr = x + t * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float v = xr[c];
#pragma unroll
        for (int i = 0; i < MAX_BRANCHES; ++i)
            if (i < br.n) v += br.scale[i] * ld((const T*)br.y[i] + t * br.stride[i] + c);
        if (br.n) xr[c] = v;
        ss += v * v;
    }
    if (!h) return;
    const float r = rsqrtf(block_sum(ss, red) / (float)W + eps) * gain;
    for (int c = threadIdx.x; c < W; c += blockDim.x) st(h + t * W + c, xr[c] * r);
}

template <typename T>
__global__ void rms_norm_rows_kernel(const T* __restrict__ x, long x_stride,
                                     const float* __restrict__ w, T* __restrict__ out, int n,
                                     float eps) {
    __shared__ float red[16];
    const long t = blockIdx.x;
    const T* xr = x + t * x_stride;
    float ss = 0.f;
    for (int c = threadIdx.x; c < n; c += blockDim.x) { const float v = ld(xr + c); ss += v * v; }
    const float r = rsqrtf(block_sum(ss, red) / (float)n + eps);
    for (int c = threadIdx.x; c < n; c += blockDim.x) st(out + t * n + c, ld(xr + c) * r * w[c]);
}

// q row [nq] normed in place with qw (when given); k row [nk] normed with kw (when given) into
// k_cache[slot]; v row [nv] into v_cache[slot].  Caches contiguous [slot, G, D|E], so a token's
// heads are one run of nk / nv numbers.
template <typename T>
__global__ void row_norm_store_kernel(T* __restrict__ q, const T* __restrict__ k,
                                      const T* __restrict__ v, long row_stride,
                                      const float* __restrict__ qw, const float* __restrict__ kw,
                                      float eps, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                      const int* __restrict__ slot_mapping, int nq, int nk, int nv) {
    __shared__ float red[16];
    const long t = blockIdx.x;
    const long slot = slot_mapping ? slot_mapping[t] : -1;
    const bool store = slot >= 0 && k_cache;
    T* qr = q + t * row_stride;
    const T* kr = k + t * row_stride;
    const T* vr = v + t * row_stride;
    if (qw) {
        float ss = 0.f;
        for (int c = threadIdx.x; c < nq; c += blockDim.x) { const float a = ld(qr + c); ss += a * a; }
        const float r = rsqrtf(block_sum(ss, red) / (float)nq + eps);
        for (int c = threadIdx.x; c < nq; c += blockDim.x) st(qr + c, ld(qr + c) * r * qw[c]);
    }
    float rk = 1.f;
    if (kw) {
        float ss = 0.f;
        for (int c = threadIdx.x; c < nk; c += blockDim.x) { const float a = ld(kr + c); ss += a * a; }
        rk = rsqrtf(block_sum(ss, red) / (float)nk + eps);
    }
    if (!store) return;
    for (int c = threadIdx.x; c < nk; c += blockDim.x)
        st(k_cache + slot * nk + c, kw ? ld(kr + c) * rk * kw[c] : ld(kr + c));
    for (int c = threadIdx.x; c < nv; c += blockDim.x) st(v_cache + slot * nv + c, ld(vr + c));
}

// Per token: c = rmsnorm(dkv[0:R]) * w;  K cache row = [c | rot(dkv[R:R+P])], V cache row = c
// (when a separate V cache is given);
// out[t, h] = [q_abs[h, t, 0:R] | rot(q[t, h, D:D+P])].  rot: entry i < dims/2 pairs with entry
// i + dims/2, angle = position * inv_freq[i] (fp32 product), entries from dims on unchanged.
template <typename T>
__global__ void latent_rope_store_kernel(const T* __restrict__ q_abs, const T* __restrict__ q,
                                         long q_row, const T* __restrict__ dkv, long dkv_row,
                                         const float* __restrict__ w, float eps,
                                         const int* __restrict__ positions,
                                         const float* __restrict__ inv_freq, int dims,
                                         T* __restrict__ k_cache, T* __restrict__ v_cache,
                                         const int* __restrict__ slot_mapping, T* __restrict__ out,
                                         long T_, int H, int D, int P, int R) {
    extern __shared__ float sm[];            // [dims/2] cos, [dims/2] sin, then 16 for sums
    const int half = dims / 2;
    float* cs = sm;
    float* sn = sm + half;
    float* red = sm + 2 * half;
    const long t = blockIdx.x;
    const long slot = slot_mapping ? slot_mapping[t] : -1;
    const bool store = slot >= 0 && k_cache;
    const float p = (float)positions[t];
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        float s_, c_;
        sincosf(p * inv_freq[i], &s_, &c_);
        cs[i] = c_; sn[i] = s_;
    }
    const T* lr = dkv + t * dkv_row;
    float ss = 0.f;
    for (int c = threadIdx.x; c < R; c += blockDim.x) { const float a = ld(lr + c); ss += a * a; }
    const float r = rsqrtf(block_sum(ss, red) / (float)R + eps);     // (its barriers publish cs / sn)
    const int DK = R + P;
    if (store) {
        for (int c = threadIdx.x; c < R; c += blockDim.x) {
            const float a = ld(lr + c) * r * w[c];
            st(k_cache + slot * DK + c, a);
            if (v_cache) st(v_cache + slot * R + c, a);   // null: values are read from the key rows
        }
        for (int i = threadIdx.x; i < P; i += blockDim.x) {
            float a;
            if (i < half) a = ld(lr + R + i) * cs[i] - ld(lr + R + i + half) * sn[i];
            else if (i < dims) a = ld(lr + R + i) * cs[i - half] + ld(lr + R + i - half) * sn[i - half];
            else a = ld(lr + R + i);
            st(k_cache + slot * DK + R + i, a);
        }
    }
    for (int j = threadIdx.x; j < H * DK; j += blockDim.x) {
        const int hh = j / DK, c = j - hh * DK;
        float a;
        if (c < R) a = ld(q_abs + ((long)hh * T_ + t) * R + c);
        else {
            const T* qr = q + t * q_row + (long)hh * (D + P) + D;
            const int i = c - R;
            if (i < half) a = ld(qr + i) * cs[i] - ld(qr + i + half) * sn[i];
            else if (i < dims) a = ld(qr + i) * cs[i - half] + ld(qr + i - half) * sn[i - half];
            else a = ld(qr + i);
        }
        st(out + t * (long)(H * DK) + j, a);
    }
}

__device__ __forceinline__ float xielu_(float z, float above, float below) {
    return z > 0.f ? above * z * z + 0.5f * z : below * (expm1f(z) - z) + 0.5f * z;
}

// act = above z^2 + z/2 (z > 0);  below (e^z - 1 - z) + z/2 (z <= 0).  u rows strided, act dense.
// VEC consecutive columns per thread (VEC = 8: rows and row starts are whole 16-byte runs).
template <typename T, int VEC>
__global__ void xielu_kernel(const T* __restrict__ u, long u_stride, T* __restrict__ act, int n,
                             float above, float below) {
    const long t = blockIdx.y;
    for (int c = (blockIdx.x * blockDim.x + threadIdx.x) * VEC; c < n; c += gridDim.x * blockDim.x * VEC) {
        if constexpr (VEC == 8) {
            float z[8];
            load_run<T, 8>(u + t * u_stride + c, z);
#pragma unroll
            for (int j = 0; j < 8; ++j) z[j] = xielu_(z[j], above, below);
            store_run8<T>(act + t * (long)n + c, z);
        } else {
            st(act + t * (long)n + c, xielu_(ld(u + t * u_stride + c), above, below));
        }
    }
}

// y = (o + skip[h] x) silu(z) over the row's H*E columns, kept in LDS; each of `groups` equal
// parts divided by its own root mean square; times w.
template <typename T>
__global__ void gated_group_norm_kernel(const float* __restrict__ o, const float* __restrict__ x,
                                        const float* __restrict__ skip, const T* __restrict__ z,
                                        long z_stride, const float* __restrict__ w,
                                        T* __restrict__ out, int H, int E, int groups, float eps) {
    extern __shared__ float sm[];            // [H*E] y, [groups] scales, 16 for sums
    const int n = H * E, part = n / groups;
    float* y = sm;
    float* gs = sm + n;
    float* red = gs + groups;
    const long t = blockIdx.x;
    for (int g = 0; g < groups; ++g) {
        float ss = 0.f;
        for (int c = g * part + threadIdx.x; c < (g + 1) * part; c += blockDim.x) {
            const float a = (o[t * n + c] + skip[c / E] * x[t * n + c]) * siluf_(ld(z + t * z_stride + c));
            y[c] = a;
            ss += a * a;
        }
        const float tot = block_sum(ss, red);
        if (threadIdx.x == 0) gs[g] = rsqrtf(tot / (float)part + eps);
    }
    __syncthreads();
    for (int c = threadIdx.x; c < n; c += blockDim.x) st(out + t * (long)n + c, y[c] * gs[c / part] * w[c]);
}

// out[t, h*E + e] = o[t, h, e] * sigmoid(gate[t, h*E + e]); o with strides (o_t, o_h, 1).
template <typename T, int VEC>
__global__ void sigmoid_gate_kernel(const T* __restrict__ o, long o_t, long o_h,
                                    const T* __restrict__ gate, long gate_stride,
                                    T* __restrict__ out, int H, int E) {
    const long t = blockIdx.y;
    const int n = H * E;
    for (int c = (blockIdx.x * blockDim.x + threadIdx.x) * VEC; c < n; c += gridDim.x * blockDim.x * VEC) {
        const int hh = c / E, e = c - hh * E;
        if constexpr (VEC == 8) {                       // E % 8 == 0: a run stays inside one head
            float a[8], g[8];
            load_run<T, 8>(o + t * o_t + hh * o_h + e, a);
            load_run<T, 8>(gate + t * gate_stride + c, g);
#pragma unroll
            for (int j = 0; j < 8; ++j) a[j] *= sigmoidf_(g[j]);
            store_run8<T>(out + t * (long)n + c, a);
        } else {
            st(out + t * (long)n + c, ld(o + t * o_t + hh * o_h + e) * sigmoidf_(ld(gate + t * gate_stride + c)));
        }
    }
}

static inline int threads_for(int n) { return n >= 1024 ? 512 : n >= 256 ? 256 : n > 64 ? 128 : 64; }

extern "C" {

// ys / strides / scales: nb (<= 4) branches of the activation type; h may be null.
int hyb_residual_sum_norm(void* x, const void* const* ys, const long* strides, const float* scales,
                          int nb, float gain, void* h, long T_, int W, float eps, int dt,
                          hipStream_t s) {
    if (T_ <= 0) return 0;
    if (nb < 0 || nb > MAX_BRANCHES) return 1;
    if (!nb && !h) return 0;
    Branches br;
    br.n = nb;
    for (int i = 0; i < MAX_BRANCHES; ++i) {
        br.y[i] = i < nb ? ys[i] : nullptr;
        br.stride[i] = i < nb ? strides[i] : 0;
        br.scale[i] = i < nb ? scales[i] : 0.f;
    }
    HYB_DISPATCH(dt, hipLaunchKernelGGL(residual_sum_norm_kernel<T>, dim3(T_), dim3(threads_for(W)),
                                        0, s, (float*)x, br, gain, (T*)h, W, eps));
    return HYB_LAUNCH_OK();
}

int hyb_rms_norm_rows(const void* x, long x_stride, const void* w, void* out, long T_, int n,
                      float eps, int dt, hipStream_t s) {
    if (T_ <= 0 || n <= 0) return 0;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(rms_norm_rows_kernel<T>, dim3(T_), dim3(threads_for(n)), 0, s,
                                        (const T*)x, x_stride, (const float*)w, (T*)out, n, eps));
    return HYB_LAUNCH_OK();
}

int hyb_row_norm_store(void* q, const void* k, const void* v, long row_stride, const void* qw,
                       const void* kw, float eps, void* k_cache, void* v_cache,
                       const void* slot_mapping, long T_, int nq, int nk, int nv, int dt,
                       hipStream_t s) {
    if (T_ <= 0) return 0;
    if ((qw == nullptr) != (kw == nullptr)) return 1;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(row_norm_store_kernel<T>, dim3(T_),
                                        dim3(threads_for(nq > nk + nv ? nq : nk + nv)), 0, s, (T*)q,
                                        (const T*)k, (const T*)v, row_stride, (const float*)qw,
                                        (const float*)kw, eps, (T*)k_cache, (T*)v_cache,
                                        (const int*)slot_mapping, nq, nk, nv));
    return HYB_LAUNCH_OK();
}

int hyb_latent_rope_store(const void* q_abs, const void* q, long q_row, const void* dkv,
                          long dkv_row, const void* w, float eps, const void* positions,
                          const void* inv_freq, int dims, void* k_cache, void* v_cache,
                          const void* slot_mapping, void* out, long T_, int H, int D, int P, int R,
                          int dt, hipStream_t s) {
    if (T_ <= 0) return 0;
    if (dims < 0 || (dims & 1) || dims > P || H <= 0 || R <= 0) return 1;
    const size_t lds = (dims + 16) * sizeof(float);
    if (lds > 64 * 1024) return 1;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(latent_rope_store_kernel<T>, dim3(T_),
                                        dim3(threads_for(H * (R + P))), lds, s, (const T*)q_abs,
                                        (const T*)q, q_row, (const T*)dkv, dkv_row, (const float*)w,
                                        eps, (const int*)positions, (const float*)inv_freq, dims,
                                        (T*)k_cache, (T*)v_cache, (const int*)slot_mapping, (T*)out,
                                        T_, H, D, P, R));
    return HYB_LAUNCH_OK();
}

// rows of n elements, `stride` apart, can be walked in aligned runs of eight
static inline bool runs_of_8(const void* p, long stride, int n, int dt) {
    return n % 8 == 0 && stride % 8 == 0 && (size_t)p % 16 == 0;
}

int hyb_xielu(const void* u, long u_stride, void* act, long T_, int n, float above, float below,
              int dt, hipStream_t s) {
    if (T_ <= 0 || n <= 0) return 0;
    const bool vec = runs_of_8(u, u_stride, n, dt) && runs_of_8(act, n, n, dt);
    const int need = (n / (vec ? 8 : 1) + 255) / 256;
    const int bx = need > 64 ? 64 : need;
    for (long t0 = 0; t0 < T_; t0 += 65535) {          // blockIdx.y holds at most 65535 rows
        const long nrow = T_ - t0 < 65535 ? T_ - t0 : 65535;
#define XIE(VEC)                                                                                   \
        HYB_DISPATCH(dt, hipLaunchKernelGGL((xielu_kernel<T, VEC>), dim3(bx, nrow), dim3(256), 0, s, \
                                            (const T*)u + t0 * u_stride, u_stride,                 \
                                            (T*)act + t0 * (long)n, n, above, below))
        if (vec) XIE(8); else XIE(1);
#undef XIE
    }
    return HYB_LAUNCH_OK();
}

int hyb_gated_group_norm(const void* o, const void* x, const void* skip, const void* z,
                         long z_stride, const void* w, void* out, long T_, int H, int E, int groups,
                         float eps, int dt, hipStream_t s) {
    if (T_ <= 0) return 0;
    const int n = H * E;
    if (groups < 1 || n % groups || groups > 1024) return 1;
    const size_t lds = ((size_t)n + groups + 16) * sizeof(float);
    if (lds > 64 * 1024) return 1;
    HYB_DISPATCH(dt, hipLaunchKernelGGL(gated_group_norm_kernel<T>, dim3(T_),
                                        dim3(threads_for(n / groups)), lds, s, (const float*)o,
                                        (const float*)x, (const float*)skip, (const T*)z, z_stride,
                                        (const float*)w, (T*)out, H, E, groups, eps));
    return HYB_LAUNCH_OK();
}

int hyb_sigmoid_gate(const void* o, long o_t, long o_h, const void* gate, long gate_stride,
                     void* out, long T_, int H, int E, int dt, hipStream_t s) {
    if (T_ <= 0 || H * E <= 0) return 0;
    const bool vec = E % 8 == 0 && o_h % 8 == 0 && runs_of_8(o, o_t, E, dt) &&
                     runs_of_8(gate, gate_stride, H * E, dt) && runs_of_8(out, H * E, H * E, dt);
    const int need = (H * E / (vec ? 8 : 1) + 255) / 256;
    const int bx = need > 64 ? 64 : need;
    for (long t0 = 0; t0 < T_; t0 += 65535) {
        const long nrow = T_ - t0 < 65535 ? T_ - t0 : 65535;
#define SGT(VEC)                                                                                   \
        HYB_DISPATCH(dt, hipLaunchKernelGGL((sigmoid_gate_kernel<T, VEC>), dim3(bx, nrow), dim3(256), \
                                            0, s, (const T*)o + t0 * o_t, o_t, o_h,                \
                                            (const T*)gate + t0 * gate_stride, gate_stride,        \
                                            (T*)out + t0 * (long)(H * E), H, E))
        if (vec) SGT(8); else SGT(1);
#undef SGT
    }
    return HYB_LAUNCH_OK();
}

}  // extern "C"
