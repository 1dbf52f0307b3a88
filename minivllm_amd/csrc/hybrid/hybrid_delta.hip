// Gated delta rule: preparation of a step's tokens (short causal convolution + silu on q / k / v,
// unit vectors, beta and decay) and the recurrence itself, for prefill portions and single
// decode tokens alike.  Everything here is fp32 except the projection outputs it reads.
// The state-space form (`ssd`: a convolution with bias, q / k as convolved, beta = the step size
// softplus(a + dt_bias), decay = exp(-exp(A_log) beta)) and the update without the correction
// term (`DELTA` false: u = beta v) make the same two kernels run a Mamba-2 style mixer.
//
// Sequence layout: `cu_q` [B+1] rows of each sequence (null: row b is sequence b), `positions`
// (a sequence's first row holds the position its portion starts at; 0 = start from zeros),
// `slots` [B] state slot per sequence (< 0: unused row of a padded batch), `row_seq` [T] the
// sequence of each row in prefill form (< 0: no sequence).
#include "hybrid_common.h"

using namespace hyb;

constexpr int MAX_TAPS = 32;

// One workgroup per token row.  proj row = [q (G*D) | k (G*D) | v (H*E) | ... | b (H) | ...];
// the three convolved blocks are contiguous at the row's start (C = 2GD + HE channels).  The
// decay's pre-activation `a` is a row of its own tensor (or a view into proj): DC entries per
// head, DC = 1 (a decay per head) or D (one per head and key channel); dt_bias has H * DC
// entries, decay out [T, H * DC].
// conv_w [C, taps] (q, k, v rows stacked), conv_state [slots, taps-1, C].
template <typename T, int TAPS>
__global__ void delta_prepare_kernel(const T* __restrict__ proj, long row_stride, int b_off,
                                     const T* __restrict__ a, long a_row, int DC,
                                     const float* __restrict__ conv_w, int taps_rt,
                                     const float* __restrict__ conv_b, int ssd,
                                     const float* __restrict__ a_log,
                                     const float* __restrict__ dt_bias,
                                     const float* __restrict__ conv_state,
                                     const int* __restrict__ cu_q, const int* __restrict__ positions,
                                     const int* __restrict__ slots, const int* __restrict__ row_seq,
                                     float* __restrict__ qn, float* __restrict__ kn,
                                     float* __restrict__ vv, float* __restrict__ beta,
                                     float* __restrict__ decay, int H, int G, int D, int E,
                                     int vec8) {
    extern __shared__ float y[];                     // [2GD] convolved + silu q, k
    const int taps = TAPS ? TAPS : taps_rt;          // TAPS > 0: known at compile time (unrolled)
    const long t = blockIdx.x;
    const int b = row_seq ? row_seq[t] : (int)t;
    if (b < 0) return;
    const int slot = slots[b];
    if (slot < 0) return;
    const long first = cu_q ? cu_q[b] : t;           // the sequence's first row in this step
    const int i = (int)(t - first);                  // index inside the portion
    const bool has_past = positions[first] > 0;
    const int C = 2 * G * D + H * E, GD = G * D;
    const float* tail = conv_state + (long)slot * (taps - 1) * C;
    if (TAPS > 0 && vec8) {
        // eight channels per thread and step, every load of the step issued before its first use:
        // one 16-byte (bf16) load per tap and the channels' taps as whole rows of the tap table
        constexpr int NT = TAPS ? TAPS : 1;
        for (int c = threadIdx.x * 8; c < C; c += blockDim.x * 8) {
            float x[NT][8], w[8][NT];
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const int back = NT - 1 - j;
                if (i - back >= 0) load_run<T, 8>(proj + (t - back) * row_stride + c, x[j]);
                else if (has_past) load_run<float, 8>(tail + (long)(NT - 1 + i - back) * C + c, x[j]);
                else {
#pragma unroll
                    for (int z = 0; z < 8; ++z) x[j][z] = 0.f;
                }
            }
#pragma unroll
            for (int z = 0; z < 8; ++z)
#pragma unroll
                for (int j = 0; j < NT; ++j) w[z][j] = conv_w[(long)(c + z) * NT + j];
            float acc[8];
#pragma unroll
            for (int z = 0; z < 8; ++z) {
                float a = conv_b ? conv_b[c + z] : 0.f;
#pragma unroll
                for (int j = 0; j < NT; ++j) a += x[j][z] * w[z][j];
                acc[z] = siluf_(a);
            }
            float* dst = (c < 2 * GD) ? y + c : vv + t * (long)(H * E) + (c - 2 * GD);
            *reinterpret_cast<float4*>(dst) = make_float4(acc[0], acc[1], acc[2], acc[3]);
            *reinterpret_cast<float4*>(dst + 4) = make_float4(acc[4], acc[5], acc[6], acc[7]);
        }
    } else
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
        float acc = conv_b ? conv_b[c] : 0.f;
        for (int j = 0; j < taps; ++j) {             // tap j reads the input `taps-1-j` tokens back
            const int back = taps - 1 - j;
            float x;
            if (i - back >= 0) x = ld(proj + (t - back) * row_stride + c);
            else x = has_past ? tail[(long)(taps - 1 + i - back) * C + c] : 0.f;
            acc += x * conv_w[(long)c * taps + j];
        }
        acc = siluf_(acc);
        if (c < 2 * GD) y[c] = acc;
        else vv[t * (long)(H * E) + (c - 2 * GD)] = acc;
    }
    __syncthreads();
    const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1), nw = blockDim.x / kWave;
    for (int hd = wave; hd < 2 * G; hd += nw) {      // heads of q (0..G-1) then of k
        const float* src = y + hd * D;
        float s = 0.f;
        for (int d = lane; d < D; d += kWave) s += src[d] * src[d];
        float r = ssd ? 1.f : rsqrtf(wave_sum(s) + 1e-6f);
        float* dst;
        if (hd < G) { if (!ssd) r *= rsqrtf((float)D); dst = qn + (t * G + hd) * (long)D; }
        else dst = kn + (t * G + hd - G) * (long)D;
        for (int d = lane; d < D; d += kWave) dst[d] = src[d] * r;
    }
    if (!ssd)
        for (int h = threadIdx.x; h < H; h += blockDim.x)
            beta[t * H + h] = sigmoidf_(ld(proj + t * row_stride + b_off + h));
    for (int c = threadIdx.x; c < H * DC; c += blockDim.x) {
        const float sp = softplusf_(ld(a + t * a_row + c) + dt_bias[c]);
        if (ssd) beta[t * H + c] = sp;               // DC == 1: the step size of head c
        decay[t * (long)(H * DC) + c] = expf(-expf(a_log[c / DC]) * sp);
    }
}

// One workgroup per sequence: the convolution inputs of the portion's last taps-1 tokens become
// the slot's tail (older entries shift when the portion is shorter).  Runs after delta_prepare.
template <typename T>
__global__ void delta_conv_tail_kernel(const T* __restrict__ proj, long row_stride, int taps,
                                       float* __restrict__ conv_state,
                                       const int* __restrict__ cu_q,
                                       const int* __restrict__ positions,
                                       const int* __restrict__ slots, int C) {
    const int b = blockIdx.x;
    const int slot = slots[b];
    if (slot < 0 || taps <= 1) return;
    const long first = cu_q ? cu_q[b] : b;
    const int n = cu_q ? cu_q[b + 1] - cu_q[b] : 1;
    if (n <= 0) return;
    const bool has_past = positions[first] > 0;
    float* tail = conv_state + (long)slot * (taps - 1) * C;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
        float nv[MAX_TAPS];
#pragma unroll
        for (int j = 0; j < MAX_TAPS - 1; ++j) {
            if (j < taps - 1) {
                const int i = n - (taps - 1) + j;    // index inside the portion, may be negative
                if (i >= 0) nv[j] = ld(proj + (first + i) * row_stride + c);
                else nv[j] = has_past ? tail[(long)(taps - 1 + i) * C + c] : 0.f;
            }
        }
#pragma unroll
        for (int j = 0; j < MAX_TAPS - 1; ++j)
            if (j < taps - 1) tail[(long)j * C + c] = nv[j];
    }
}

// The recurrence.  A state column S[:, e] evolves independently of the others:
//   u_e = beta (v_e - g sum_d S[d,e] k_d);  S[d,e] <- g S[d,e] + k_d u_e;  o_e = sum_d S[d,e] q_d
// so a column is owned by 4 neighbouring lanes, lane r holding d in [r*NR, (r+1)*NR) in
// registers (D <= 4*NR, missing d padded with zeros); the two sums over d close with two
// exchanges inside the quad.  Workgroup = 64 columns of one (sequence, head).  The tokens'
// operands (k, q of the head: shared by all columns; v of the 64 columns; beta, decay) are
// staged through LDS in chunks of CT tokens, double-buffered: the next chunk's global loads are
// in flight while the current chunk's steps run, and a step reads its k / q slice with 16-byte
// LDS reads (per-lane global loads of these shared vectors were what bound the first version).
template <int NR> struct ScanChunk { static constexpr int tokens = NR >= 64 ? 8 : 16; };

template <int NR, bool DELTA>
__global__ void __launch_bounds__(256)
delta_scan_kernel(const float* __restrict__ qn, const float* __restrict__ kn,
                  const float* __restrict__ vv, const float* __restrict__ beta,
                  const float* __restrict__ decay, float* __restrict__ state,
                  const int* __restrict__ cu_q, const int* __restrict__ positions,
                  const int* __restrict__ slots, float* __restrict__ o, int H, int G, int D, int E) {
    constexpr int CT = ScanChunk<NR>::tokens;
    constexpr int RS = NR + 4;                 // padded slice: the 4 lanes of a quad hit 4 bank groups
    constexpr int KQ = CT * 4 * RS;            // floats of one k (or q) chunk image
    constexpr int BUF = 2 * KQ + CT * 64 + 2 * CT;
    constexpr int NLD = (2 * CT * 4 * NR + CT * 64 + 2 * CT + 255) / 256;   // staged floats per thread
    extern __shared__ float sm[];
    const int b = blockIdx.x, h = blockIdx.y;
    const int slot = slots[b];
    if (slot < 0) return;
    const long first = cu_q ? cu_q[b] : b;
    const int n = cu_q ? cu_q[b + 1] - cu_q[b] : 1;
    if (n <= 0) return;
    const int tid = threadIdx.x, r = tid & 3, c = tid >> 2;
    const int e0 = blockIdx.z * 64, e = e0 + c;
    const bool col = e < E;
    const int g = h / (H / G);
    const int d0 = r * NR;
    float S[NR];
    float* sp = state + (((long)slot * H + h) * D) * E + (col ? e : 0);
    const bool has_past = positions[first] > 0;
#pragma unroll
    for (int i = 0; i < NR; ++i)
        S[i] = (has_past && col && d0 + i < D) ? sp[(long)(d0 + i) * E] : 0.f;

    // staging: item j of a chunk = one float of k, q (padded to 4*NR per token), v, beta, decay
    auto fetch = [&](int chunk, float* reg) {
        const long t0 = first + (long)chunk * CT;
        const int nt = min(CT, n - chunk * CT);
#pragma unroll
        for (int x = 0; x < NLD; ++x) {
            const int j = tid + x * 256;
            float v = 0.f;
            if (j < 2 * CT * 4 * NR) {
                const int which = j / (CT * 4 * NR), jj = j - which * (CT * 4 * NR);
                const int tok = jj / (4 * NR), d = jj - tok * (4 * NR);
                if (tok < nt && d < D)
                    v = (which ? qn : kn)[((t0 + tok) * G + g) * (long)D + d];
            } else if (j < 2 * CT * 4 * NR + CT * 64) {
                const int jj = j - 2 * CT * 4 * NR, tok = jj >> 6, cc = jj & 63;
                if (tok < nt && e0 + cc < E) v = vv[((t0 + tok) * H + h) * (long)E + e0 + cc];
            } else if (j < 2 * CT * 4 * NR + CT * 64 + 2 * CT) {
                const int jj = j - 2 * CT * 4 * NR - CT * 64, tok = jj % CT;
                if (tok < nt) v = (jj < CT ? beta : decay)[(t0 + tok) * H + h];
            }
            reg[x] = v;
        }
    };
    auto stash = [&](const float* reg, float* buf) {
#pragma unroll
        for (int x = 0; x < NLD; ++x) {
            const int j = tid + x * 256;
            if (j < 2 * CT * 4 * NR) {
                const int which = j / (CT * 4 * NR), jj = j - which * (CT * 4 * NR);
                const int tok = jj / (4 * NR), d = jj - tok * (4 * NR);
                buf[which * KQ + (tok * 4 + d / NR) * RS + d % NR] = reg[x];
            } else if (j < 2 * CT * 4 * NR + CT * 64 + 2 * CT) {
                buf[2 * KQ + j - 2 * CT * 4 * NR] = reg[x];
            }
        }
    };
    float reg[NLD];
    fetch(0, reg);
    stash(reg, sm);
    __syncthreads();
    const int nchunks = (n + CT - 1) / CT;
    for (int ch = 0; ch < nchunks; ++ch) {
        const float* buf = sm + (ch & 1) * BUF;
        if (ch + 1 < nchunks) fetch(ch + 1, reg);
        const int nt = min(CT, n - ch * CT);
#pragma unroll 2
        for (int tok = 0; tok < nt; ++tok) {
            const float4* kp = reinterpret_cast<const float4*>(buf + (tok * 4 + r) * RS);
            const float4* qp = reinterpret_cast<const float4*>(buf + KQ + (tok * 4 + r) * RS);
            const float ve = buf[2 * KQ + tok * 64 + c];
            const float bt = buf[2 * KQ + CT * 64 + tok], gd = buf[2 * KQ + CT * 64 + CT + tok];
            float4 k4[NR / 4], q4[NR / 4];
#pragma unroll
            for (int i = 0; i < NR / 4; ++i) { k4[i] = kp[i]; q4[i] = qp[i]; }
            // four partial sums each: a single chain of NR dependent FMAs would be what a step
            // waits for (one wave per SIMD: nobody else fills the gaps)
            float u = bt * ve;
            if constexpr (DELTA) {
                float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
                for (int i = 0; i < NR / 4; ++i) {
                    d0 += S[4 * i] * k4[i].x; d1 += S[4 * i + 1] * k4[i].y;
                    d2 += S[4 * i + 2] * k4[i].z; d3 += S[4 * i + 3] * k4[i].w;
                }
                float dot = (d0 + d1) + (d2 + d3);
                dot += __shfl_xor(dot, 1, kWave);
                dot += __shfl_xor(dot, 2, kWave);
                u = bt * (ve - gd * dot);
            }
            float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
            for (int i = 0; i < NR / 4; ++i) {
                S[4 * i] = gd * S[4 * i] + k4[i].x * u;         o0 += S[4 * i] * q4[i].x;
                S[4 * i + 1] = gd * S[4 * i + 1] + k4[i].y * u; o1 += S[4 * i + 1] * q4[i].y;
                S[4 * i + 2] = gd * S[4 * i + 2] + k4[i].z * u; o2 += S[4 * i + 2] * q4[i].z;
                S[4 * i + 3] = gd * S[4 * i + 3] + k4[i].w * u; o3 += S[4 * i + 3] * q4[i].w;
            }
            float out = (o0 + o1) + (o2 + o3);
            out += __shfl_xor(out, 1, kWave);
            out += __shfl_xor(out, 2, kWave);
            if (col && r == 0) o[((first + ch * CT + tok) * H + h) * (long)E + e] = out;
        }
        if (ch + 1 < nchunks) stash(reg, sm + ((ch + 1) & 1) * BUF);
        __syncthreads();
    }
    if (col) {
#pragma unroll
        for (int i = 0; i < NR; ++i)
            if (d0 + i < D) sp[(long)(d0 + i) * E] = S[i];
    }
}

template <int NR, bool DELTA>
static void launch_scan(dim3 grid, hipStream_t s, const void* qn, const void* kn, const void* vv,
                        const void* beta, const void* decay, void* state, const void* cu_q,
                        const void* positions, const void* slots, void* o, int H, int G, int D, int E) {
    constexpr int CT = ScanChunk<NR>::tokens;
    constexpr int BUF = 2 * CT * 4 * (NR + 4) + CT * 64 + 2 * CT;
    hipLaunchKernelGGL((delta_scan_kernel<NR, DELTA>), grid, dim3(256), 2 * BUF * sizeof(float), s,
                       (const float*)qn, (const float*)kn, (const float*)vv, (const float*)beta,
                       (const float*)decay, (float*)state, (const int*)cu_q, (const int*)positions,
                       (const int*)slots, (float*)o, H, G, D, E);
}

extern "C" {

int hyb_delta_prepare(const void* proj, long row_stride, int b_off, const void* a, long a_row,
                      int DC, const void* conv_w, int taps, const void* conv_b, int ssd,
                      const void* a_log, const void* dt_bias, void* conv_state,
                      const void* cu_q, const void* positions, const void* slots,
                      const void* row_seq, void* qn, void* kn, void* vv, void* beta, void* decay,
                      long T_, int B, int H, int G, int D, int E, int dt, hipStream_t s) {
    if (T_ <= 0) return 0;
    if (taps < 1 || taps > MAX_TAPS || H % G || (DC != 1 && DC != D) || (ssd && DC != 1)) return 1;
    const int C = 2 * G * D + H * E;
    const size_t lds = 2 * (size_t)G * D * sizeof(float);
    if (lds > 64 * 1024) return 1;
    const int vec8 = (G * D) % 8 == 0 && (H * E) % 8 == 0 && row_stride % 8 == 0 &&
                     (size_t)proj % 16 == 0 && (size_t)conv_state % 16 == 0 && (size_t)vv % 16 == 0;
#define PREP(TAPS)                                                                                 \
    HYB_DISPATCH(dt, hipLaunchKernelGGL((delta_prepare_kernel<T, TAPS>), dim3(T_),                 \
                                        dim3(C >= 2048 && T_ <= 1024 ? 1024 : 256), lds, s,        \
                                        (const T*)proj, row_stride, b_off, (const T*)a, a_row, DC, \
                                        (const float*)conv_w, taps, (const float*)conv_b, ssd,     \
                                        (const float*)a_log,                                       \
                                        (const float*)dt_bias, (const float*)conv_state,           \
                                        (const int*)cu_q, (const int*)positions, (const int*)slots,\
                                        (const int*)row_seq, (float*)qn, (float*)kn, (float*)vv,   \
                                        (float*)beta, (float*)decay, H, G, D, E, vec8))
    if (taps == 4) PREP(4);
    else if (taps == 3) PREP(3);
    else if (taps == 2) PREP(2);
    else PREP(0);
#undef PREP
    if (hipGetLastError() != hipSuccess) return 2;
    if (taps > 1) {
        HYB_DISPATCH(dt, hipLaunchKernelGGL(delta_conv_tail_kernel<T>, dim3(B, (C + 255) / 256),
                                            dim3(256), 0, s,
                                            (const T*)proj, row_stride, taps, (float*)conv_state,
                                            (const int*)cu_q, (const int*)positions,
                                            (const int*)slots, C));
    }
    return HYB_LAUNCH_OK();
}

int hyb_delta_scan(const void* qn, const void* kn, const void* vv, const void* beta,
                   const void* decay, void* state, const void* cu_q, const void* positions,
                   const void* slots, void* o, int B, int H, int G, int D, int E, int correct,
                   hipStream_t s) {
    if (B <= 0) return 0;
    if (H % G || D > 256) return 1;
    const dim3 grid(B, H, (E + 63) / 64);
#define SCAN(NR)                                                                                       \
    do {                                                                                               \
        if (correct) launch_scan<NR, true>(grid, s, qn, kn, vv, beta, decay, state, cu_q, positions,   \
                                           slots, o, H, G, D, E);                                      \
        else launch_scan<NR, false>(grid, s, qn, kn, vv, beta, decay, state, cu_q, positions, slots,   \
                                    o, H, G, D, E);                                                    \
    } while (0)
    if (D <= 32) SCAN(8);
    else if (D <= 64) SCAN(16);
    else if (D <= 128) SCAN(32);
    else SCAN(64);
#undef SCAN
    return HYB_LAUNCH_OK();
}

}  // extern "C"
