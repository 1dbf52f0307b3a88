// Causal attention over a paged cache with a sink term in the softmax denominator, separate key
// and value head sizes, grouped query heads and an optional sigmoid gate per head.  fp32 scores,
// weights and accumulation for bfloat16 and float caches alike.  Three kernels:
//   sink_attention_tiles  - prompt portions on the matrix cores (below, second)
//   sink_attention_split  - decode rows at serving head sizes, context split over workgroups (third)
//   sink_attention_rows   - any head sizes, row by row: the reference form of the other two (first)
//
// sink_attention_rows: one workgroup (256 threads) per (query row, group of up to RC query heads
// that share a KV head).  The keys of the row's context are walked in tiles of 256: a thread scores one key of
// the tile against the RC heads (key read once), the tile's maximum and sum update the running
// softmax, then the threads switch roles and each owns output columns (head, e) whose weighted
// value sum it extends over the tile's keys (value rows read coalesced).  The running maximum
// starts at the sink and the running sum at 1 = exp(sink - sink): the sink is a key without a
// value.  Rows: a decode batch (row b = sequence b, context_lens[b] keys) or the rows of a
// prefill-form step (row_seq gives the sequence, positions[t] + 1 keys).
//
// Options of all three (struct KeyRule): no sink (sink == null: an ordinary softmax; the running
// maximum then starts at a large negative FINITE number and the sum at 0, so that no path forms
// inf - inf), a sliding window that keeps the first tokens (a query at position i sees key j <= i
// only when i - j < window or j < keep_first; keys outside are never loaded), and a distance
// penalty slope_h * (i - j) taken off the score; a multiplier per query head on the scaled score
// (temps), a tanh soft cap (score <- cap tanh(score / cap), after scale and multiplier), and pooled
// blocks behind the window: with pool = P > 0 a query at position i also sees ONE key / value row
// for every block b of P tokens with b P + P - 1 <= i - window.  Those rows live in the same
// allocations as the token rows, pool_base rows behind their start: pooled row b of a sequence is
// row pool_base + table[b / pool_rows] * pool_rows + b % pool_rows.  In the order the kernels walk
// a query's keys the pooled rows come first, then the window's tokens.
#include "hybrid_common.h"

using namespace hyb;

constexpr float NO_SINK_MAX = -1e30f;

struct KeyRule {
    int window;             // 0: every earlier key is visible
    int keep_first;
    const float* slopes;    // [H] or null
    int v_stride;           // elements from one (slot, KV head) value row to the next: E for a dense
                            // V cache, more when the value rows are the leading part of wider rows
                            // (values stored inside the key rows: v_cache then points into k_cache)
    const float* temps;     // [H] or null: multiplies the scaled score of head h
    float softcap;          // 0: none
    int pool;               // 0: no pooled blocks (needs window > 0 and keep_first == 0)
    int pool_rows;          // pooled rows per page
    long pool_base;         // first pooled row, in rows from the start of the K (and of the V) cache
    __device__ __forceinline__ float capped(float s) const {
        return softcap > 0.f ? softcap * tanhf(s / softcap) : s;
    }
    __device__ __forceinline__ float head_scale(float scale, int h) const {
        return temps ? scale * temps[h] : scale;
    }
    // pooled blocks a query that sees ctx keys without a window takes in
    __device__ __forceinline__ int pooled_for(int ctx) const {
        return (pool > 0 && ctx > window) ? (ctx - window) / pool : 0;
    }
    __device__ __forceinline__ long pooled_row(const int* table, int b) const {
        return pool_base + (long)table[b / pool_rows] * pool_rows + b % pool_rows;
    }
};

// The visible keys of a query that sees `ctx` keys without a window (its position is ctx - 1), as
// one run of virtual indices: [0, kept) are keys 0 .. kept-1, the rest the window's keys from `lo`.
struct VisibleKeys {
    int kept, lo, count;
    __device__ __forceinline__ VisibleKeys(int ctx, const KeyRule& r) {
        lo = r.window > 0 ? max(0, ctx - r.window) : 0;
        kept = r.pool > 0 ? r.pooled_for(ctx) : min(r.keep_first, lo);
        count = kept + ctx - lo;
    }
    __device__ __forceinline__ int key(int v) const { return v < kept ? v : lo + (v - kept); }
    // cache row of virtual key v (with pooled blocks the leading `kept` indices are pooled rows)
    __device__ __forceinline__ long row(int v, const int* table, int block_size, const KeyRule& r) const {
        if (r.pool > 0 && v < kept) return r.pooled_row(table, v);
        const int j = key(v);
        return (long)table[j / block_size] * block_size + j % block_size;
    }
};

constexpr int TILE = 256;
constexpr int RC = 4;       // query heads per workgroup
constexpr int NACC = 4;     // output columns per thread: (heads per workgroup) * E <= NACC * 256

template <typename T>
__global__ void __launch_bounds__(TILE)
sink_attention_rows_kernel(const T* __restrict__ q, long q_row, long q_head,
                           const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                           const int* __restrict__ block_tables, int max_blocks, int block_size,
                           const int* __restrict__ row_seq, const int* __restrict__ lens,
                           int len_add, const float* __restrict__ sink,
                           const T* __restrict__ gate, long gate_row, T* __restrict__ out,
                           float scale, int H, int G, int D, int E, int vec_ok, int seq_base,
                           int hpw, KeyRule rule) {
    // hpw <= RC: query heads per workgroup (fewer when a head's value row is long: the output
    // columns of a workgroup, hpw * E, are spread over NACC * TILE thread slots)
    extern __shared__ float sm[];
    const int R = H / G;
    const int chunks = (R + hpw - 1) / hpw;
    const long t = blockIdx.x;
    const int g = blockIdx.y / chunks, h0 = g * R + (blockIdx.y % chunks) * hpw;
    const int nr = min(hpw, g * R + R - h0);
    const int b = row_seq ? row_seq[t] - seq_base : (int)t;      // seq_base: first table row
    if (b < 0) return;
    const int ctx = lens[row_seq ? t : b] + len_add;
    if (ctx <= 0) return;
    const VisibleKeys vis(ctx, rule);
    const int* table = block_tables + (long)b * max_blocks;
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid & (kWave - 1);

    float* qs = sm;                           // [RC][D]
    float* ps = qs + RC * D;                  // [RC][TILE]
    float* wred = ps + RC * TILE;             // [4 waves][RC]
    float* stat = wred + 4 * RC;              // [RC] alpha, then [RC] running max, [RC] running sum
    long* rowbase = reinterpret_cast<long*>(stat + 3 * RC + 1 + ((3 * RC + 1) & 1));   // [TILE]

    for (int i = tid; i < nr * D; i += TILE) {
        const int r = i / D, d = i - r * D;
        qs[r * D + d] = ld(q + t * q_row + (long)(h0 + r) * q_head + d) * rule.head_scale(scale, h0 + r);
    }
    if (tid < RC) {
        stat[RC + tid] = tid < nr ? (sink ? sink[h0 + tid] : NO_SINK_MAX) : 0.f;   // running max
        stat[2 * RC + tid] = sink ? 1.f : 0.f;                  // running sum (the sink's term)
    }
    float slope[RC];
#pragma unroll
    for (int r = 0; r < RC; ++r) slope[r] = (rule.slopes && r < nr) ? rule.slopes[h0 + r] : 0.f;
    float acc[NACC];
#pragma unroll
    for (int a = 0; a < NACC; ++a) acc[a] = 0.f;
    __syncthreads();

    for (int j0 = 0; j0 < vis.count; j0 += TILE) {
        const bool live = j0 + tid < vis.count;
        const int j = vis.key(j0 + tid);
        float s[RC];
#pragma unroll
        for (int r = 0; r < RC; ++r) s[r] = -INFINITY;
        if (live) {
            const long slot = vis.row(j0 + tid, table, block_size, rule);
            rowbase[tid] = slot;
            const T* kr = k_cache + (slot * G + g) * (long)D;
#pragma unroll
            for (int r = 0; r < RC; ++r) s[r] = 0.f;
            if (vec_ok) {
                for (int d = 0; d < D; d += 4) {
                    float kv[4];
                    Vec4<T>::load(kr + d, kv);
#pragma unroll
                    for (int r = 0; r < RC; ++r)
                        if (r < nr) {
                            const float* qq = qs + r * D + d;
                            s[r] += kv[0] * qq[0] + kv[1] * qq[1] + kv[2] * qq[2] + kv[3] * qq[3];
                        }
                }
            } else {
                for (int d = 0; d < D; ++d) {
                    const float kv = ld(kr + d);
#pragma unroll
                    for (int r = 0; r < RC; ++r) if (r < nr) s[r] += kv * qs[r * D + d];
                }
            }
            const float dist = (float)(ctx - 1 - j);
#pragma unroll
            for (int r = 0; r < RC; ++r) s[r] = rule.capped(s[r]) - slope[r] * dist;
        }
        // tile maximum per head
#pragma unroll
        for (int r = 0; r < RC; ++r) {
            const float m = wave_max(s[r]);
            if (lane == 0) wred[wave * RC + r] = m;
        }
        __syncthreads();
        float mnew[RC];
#pragma unroll
        for (int r = 0; r < RC; ++r) {
            float m = stat[RC + r];
            for (int w = 0; w < TILE / kWave; ++w) m = fmaxf(m, wred[w * RC + r]);
            mnew[r] = m;
        }
        float psum[RC];
#pragma unroll
        for (int r = 0; r < RC; ++r) {
            const float p = (live && r < nr) ? expf(s[r] - mnew[r]) : 0.f;
            ps[r * TILE + tid] = p;
            psum[r] = wave_sum(p);
        }
        __syncthreads();                       // every thread has read wred and stat
#pragma unroll
        for (int r = 0; r < RC; ++r) if (lane == 0) wred[wave * RC + r] = psum[r];
        __syncthreads();
        if (tid < RC) {
            const int r = tid;
            const float alpha = expf(stat[RC + r] - mnew[r]);
            float l = stat[2 * RC + r] * alpha;
            for (int w = 0; w < TILE / kWave; ++w) l += wred[w * RC + r];
            stat[r] = alpha;
            stat[RC + r] = mnew[r];
            stat[2 * RC + r] = l;
        }
        __syncthreads();
        // weighted value sums: thread owns columns c = tid + a * TILE of [nr][E]
        const int n = min(TILE, vis.count - j0);
#pragma unroll
        for (int a = 0; a < NACC; ++a) {
            const int c = tid + a * TILE;
            if (c < nr * E) {
                const int r = c / E, e = c - r * E;
                float o = acc[a] * stat[r];
                const float* pr = ps + r * TILE;
                const T* vb = v_cache + (long)g * rule.v_stride + e;
                for (int jj = 0; jj < n; ++jj) o += pr[jj] * ld(vb + rowbase[jj] * (long)(G * rule.v_stride));
                acc[a] = o;
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int a = 0; a < NACC; ++a) {
        const int c = tid + a * TILE;
        if (c < nr * E) {
            const int r = c / E, e = c - r * E;
            float o = acc[a] / stat[2 * RC + r];
            if (gate) o *= sigmoidf_(ld(gate + t * gate_row + h0 + r));
            st(out + (t * H + h0 + r) * (long)E + e, o);
        }
    }
}

// ---------------------------------------------------------------------------------------
// Prompt portions: tiles on the matrix cores, everything in fp32.
//
// Workgroup = 4 waves = 128 consecutive queries of one (sequence, query head); a wave owns 32 of
// them.  Keys are walked in tiles of 32 through LDS (K tile [32][DP+1], V tile [32][EP], both
// widened to fp32 on the way in).  Scores are computed transposed, S^T = K Q^T, with
// v_mfma_f32_32x32x2_f32: a lane then holds 16 keys of ONE query (column lane%32), so the
// running maximum and sum are per-lane values (one exchange with lane^32), and the
// accumulator registers are, as they stand, the B operand of O^T += V^T P^T: register r of
// both halves of the wave names key 8(r/4) + 4(lane/32) + r%4, which is the key row the A
// operand (V^T) is read from.  The sink initialises the running maximum (sum 1).  DP / EP:
// head sizes rounded up to the template's register arrays (padding columns of K are zeroed).
typedef __attribute__((ext_vector_type(16))) float f32x16;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

// QK16 (bfloat16 caches only): the score products run as v_mfma_f32_32x32x16_bf16 on the raw
// 16-bit K tile and q rows - the operands ARE bfloat16 values, so the products are exact and the
// fp32 accumulation only differs in order from the fp32 instruction; the score scale is applied
// to the fp32 result.  Weights and weighted sums stay on the fp32 instruction.
// EXT: the instance that knows head temperatures, the soft cap and pooled rows; without it the
// kernel is compiled free of them (their state costs registers the plain form has no room for).
template <typename T, int DP, int EP, bool QK16, bool EXT>
__global__ void __launch_bounds__(256)
sink_attention_tiles_kernel(const T* __restrict__ q, long q_row, long q_head,
                            const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                            const int* __restrict__ block_tables, int max_blocks, int block_size,
                            const int* __restrict__ cu_q, const int* __restrict__ positions,
                            const float* __restrict__ sink, const T* __restrict__ gate,
                            long gate_row, T* __restrict__ out, float scale, int H, int G, int D,
                            int E, int seq0, int vec_k, int vec_v, KeyRule rule) {
    extern __shared__ float sm[];
    constexpr int KS = QK16 ? (DP + 8) / 2 : DP + 1;      // floats per K row of the LDS image
    constexpr int KSB = DP + 8;                             // (QK16) 16-bit elements per K row
    float* Ks = sm;
    uint16_t* Kb = reinterpret_cast<uint16_t*>(sm);
    float* Vs = sm + 32 * KS;
    const int b = blockIdx.x + seq0, tile = blockIdx.y, h = blockIdx.z;
    const int row0 = cu_q[b], qlen = cu_q[b + 1] - row0;
    if (tile * 128 >= qlen) return;
    const int start = positions[row0];
    const int g = h / (H / G);
    const int* table = block_tables + (long)b * max_blocks;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    const int qi = tile * 128 + wave * 32 + l32;
    const bool qok = qi < qlen;
    const int qpos = start + qi;

    const float hscale = EXT ? rule.head_scale(scale, h) : scale;
    float qreg[QK16 ? 1 : DP / 2];
    bf16x8 qv[QK16 ? DP / 16 : 1];
    {
        const T* qp = q + (long)(row0 + (qok ? qi : 0)) * q_row + (long)h * q_head;
        if constexpr (QK16) {
#pragma unroll
            for (int s = 0; s < DP / 16; ++s) {
                const int d = 16 * s + 8 * half;
                uint4 raw = make_uint4(0, 0, 0, 0);
                if (qok && d < D) raw = *reinterpret_cast<const uint4*>(qp + d);
                qv[s] = __builtin_bit_cast(bf16x8, raw);
            }
            for (int i = tid; i < 32 * (KSB - D); i += 256) {   // padding columns of K stay zero
                const int key = i / (KSB - D), c = D + i - key * (KSB - D);
                Kb[key * KSB + c] = 0;
            }
        } else {
#pragma unroll
            for (int s = 0; s < DP / 2; ++s) {
                const int d = 2 * s + half;
                qreg[s] = (qok && d < D) ? ld(qp + d) * hscale : 0.f;
            }
            for (int i = tid; i < 32 * (KS - D); i += 256) {      // padding columns of K stay zero
                const int key = i / (KS - D), c = D + i - key * (KS - D);
                Ks[key * KS + c] = 0.f;
            }
        }
    }
    float m = sink ? sink[h] : NO_SINK_MAX, lsum = sink ? 1.f : 0.f;
    const float slope = rule.slopes ? rule.slopes[h] : 0.f;
    f32x16 oacc[EP / 32];
#pragma unroll
    for (int eb = 0; eb < EP / 32; ++eb)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[eb][r] = 0.f;

    const int wg_ctx = start + min(qlen, tile * 128 + 128);            // keys this workgroup needs
    const bool wave_live = tile * 128 + wave * 32 < qlen;
    const int wave_last = start + min(qlen - 1, tile * 128 + wave * 32 + 31);
    // with a window: the oldest key any query of the workgroup / of the wave still sees
    const int wg_lo = rule.window > 0 ? max(0, start + tile * 128 - rule.window + 1) : 0;
    const int wave_lo = rule.window > 0 ? max(0, start + tile * 128 + wave * 32 - rule.window + 1) : 0;

    // pooled rows first (those the workgroup's last query takes in), then the tokens
    const int wg_nb = EXT ? rule.pooled_for(wg_ctx) : 0, ptiles = EXT ? (wg_nb + 31) / 32 : 0;
    const int wave_nb = EXT ? rule.pooled_for(wave_last + 1) : 0, q_nb = EXT ? rule.pooled_for(qpos + 1) : 0;
    for (int it = 0; it < ptiles + (wg_ctx + 31) / 32; ++it) {
        const bool pooled = EXT && it < ptiles;                       // (uniform)
        const int k0 = (pooled ? it : it - ptiles) * 32;
        const int k_lim = pooled ? wg_nb : wg_ctx;
        if (!pooled && k0 >= rule.keep_first && k0 + 32 <= wg_lo) continue;   // (uniform) nobody sees this tile
        auto cache_row = [&](int j) -> long {
            return pooled ? rule.pooled_row(table, j)
                          : (long)table[j / block_size] * block_size + j % block_size;
        };
        // ---- K and V tile into LDS
        if constexpr (QK16) {
            const int D8 = D >> 3;
            for (int i = tid; i < 32 * D8; i += 256) {
                const int key = i / D8, c = (i - key * D8) << 3, j = k0 + key;
                uint4 raw = make_uint4(0, 0, 0, 0);
                if (j < k_lim) {
                    const long slot = cache_row(j);
                    raw = *reinterpret_cast<const uint4*>(k_cache + (slot * G + g) * (long)D + c);
                }
                *reinterpret_cast<uint4*>(Kb + key * KSB + c) = raw;
            }
        } else if (vec_k) {
            const int D4 = D >> 2;
            for (int i = tid; i < 32 * D4; i += 256) {
                const int key = i / D4, c = (i - key * D4) << 2, j = k0 + key;
                float v4[4] = {0.f, 0.f, 0.f, 0.f};
                if (j < k_lim) {
                    const long slot = cache_row(j);
                    Vec4<T>::load(k_cache + (slot * G + g) * (long)D + c, v4);
                }
                float* dst = Ks + key * KS + c;
                dst[0] = v4[0]; dst[1] = v4[1]; dst[2] = v4[2]; dst[3] = v4[3];
            }
        } else {
            for (int i = tid; i < 32 * D; i += 256) {
                const int key = i / D, c = i - key * D, j = k0 + key;
                float v = 0.f;
                if (j < k_lim) {
                    const long slot = cache_row(j);
                    v = ld(k_cache + (slot * G + g) * (long)D + c);
                }
                Ks[key * KS + c] = v;
            }
        }
        if (vec_v) {
            const int E4 = E >> 2;
            for (int i = tid; i < 32 * E4; i += 256) {
                const int key = i / E4, c = (i - key * E4) << 2, j = k0 + key;
                float v4[4] = {0.f, 0.f, 0.f, 0.f};
                if (j < k_lim) {
                    const long slot = cache_row(j);
                    Vec4<T>::load(v_cache + (slot * G + g) * (long)rule.v_stride + c, v4);
                }
                float* dst = Vs + key * EP + c;
                dst[0] = v4[0]; dst[1] = v4[1]; dst[2] = v4[2]; dst[3] = v4[3];
            }
        } else {
            for (int i = tid; i < 32 * E; i += 256) {
                const int key = i / E, c = i - key * E, j = k0 + key;
                float v = 0.f;
                if (j < k_lim) {
                    const long slot = cache_row(j);
                    v = ld(v_cache + (slot * G + g) * (long)rule.v_stride + c);
                }
                Vs[key * EP + c] = v;
            }
        }
        __syncthreads();
        if (wave_live && (pooled ? k0 < wave_nb
                                 : (k0 <= wave_last && (k0 < rule.keep_first || k0 + 32 > wave_lo)))) {
            f32x16 sacc;
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
            if constexpr (QK16) {
                const uint16_t* ka = Kb + l32 * KSB + 8 * half;
#pragma unroll
                for (int s = 0; s < DP / 16; ++s) {
                    const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(ka + 16 * s));
                    sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qv[s], sacc, 0, 0, 0);
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) sacc[r] *= hscale;
            } else {
                const float* ka = Ks + l32 * KS + half;
#pragma unroll
                for (int s = 0; s < DP / 2; ++s)
                    sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[2 * s], qreg[s], sacc, 0, 0, 0);
            }
            float mt = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = k0 + 8 * (r >> 2) + 4 * half + (r & 3);
                const bool seen = qok && (pooled ? key < q_nb : (key <= qpos &&
                                  (rule.window <= 0 || qpos - key < rule.window || key < rule.keep_first)));
                const float v = seen ? (EXT ? rule.capped(sacc[r]) : sacc[r]) - (pooled ? 0.f : slope * (float)(qpos - key)) : -INFINITY;
                sacc[r] = v;
                mt = fmaxf(mt, v);
            }
            mt = fmaxf(mt, __shfl_xor(mt, 32, kWave));
            const float mnew = fmaxf(m, mt);
            const float alpha = expf(m - mnew);
            float ps = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = expf(sacc[r] - mnew);
                sacc[r] = p;
                ps += p;
            }
            ps += __shfl_xor(ps, 32, kWave);
            lsum = lsum * alpha + ps;
            m = mnew;
#pragma unroll
            for (int eb = 0; eb < EP / 32; ++eb) {
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[eb][r] *= alpha;
                const float* va = Vs + (4 * half) * EP + eb * 32 + l32;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    oacc[eb] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                        va[(8 * (r >> 2) + (r & 3)) * EP], sacc[r], oacc[eb], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    if (!qok) return;
    const long row = row0 + qi;
    float f = 1.f / lsum;
    if (gate) f *= sigmoidf_(ld(gate + row * gate_row + h));
    T* op = out + (row * H + h) * (long)E;
#pragma unroll
    for (int eb = 0; eb < EP / 32; ++eb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int e = eb * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
            if (e < E) st(op + e, oacc[eb][r] * f);
        }
}

template <typename T, int DP, int EP>
static int launch_tiles(const void* q, long q_row, long q_head, const void* k_cache,
                        const void* v_cache, const void* block_tables, int max_blocks,
                        int block_size, const void* cu_q, const void* positions, const void* sink,
                        const void* gate, long gate_row, void* out, float scale, int nseq,
                        int seq0, int max_q, int H, int G, int D, int E, int esize,
                        KeyRule rule, hipStream_t s) {
    const int vec_k = (D % 4 == 0) && ((size_t)k_cache % 16 == 0);
    const int vec_v = (E % 4 == 0) && (rule.v_stride % 4 == 0) && ((size_t)v_cache % 16 == 0);
    const dim3 grid(nseq, (max_q + 127) / 128, H);
#define TILES_LAUNCH_X(QK16, EXT, lds)                                                            \
    hipLaunchKernelGGL((sink_attention_tiles_kernel<T, DP, EP, QK16, EXT>), grid, dim3(256), lds, s, \
                       (const T*)q, q_row, q_head, (const T*)k_cache, (const T*)v_cache,          \
                       (const int*)block_tables, max_blocks, block_size, (const int*)cu_q,        \
                       (const int*)positions, (const float*)sink, (const T*)gate, gate_row,       \
                       (T*)out, scale, H, G, D, E, seq0, vec_k, vec_v, rule)
#define TILES_LAUNCH(QK16, lds)                                                                   \
    do { if (ext) TILES_LAUNCH_X(QK16, true, lds); else TILES_LAUNCH_X(QK16, false, lds); } while (0)
    const bool ext = rule.temps || rule.softcap > 0.f || rule.pool > 0;
    if constexpr (sizeof(T) == 2) {
        // 16-bit caches: score products on the bf16 instruction when rows are 16-byte addressable
        if (D % 16 == 0 && (size_t)k_cache % 16 == 0 && (size_t)q % 16 == 0 && q_row % 8 == 0 &&
            q_head % 8 == 0) {
            TILES_LAUNCH(true, (32 * ((DP + 8) / 2) + 32 * EP) * sizeof(float));
            return HYB_LAUNCH_OK();
        }
    }
    TILES_LAUNCH(false, (32 * (DP + 1) + 32 * EP) * sizeof(float));
#undef TILES_LAUNCH
#undef TILES_LAUNCH_X
    return HYB_LAUNCH_OK();
}

// ---------------------------------------------------------------------------------------
// Decode rows at serving sizes: the context is split over workgroups and every K / V row is
// read by 16 neighbouring lanes with 16-byte (bf16: EPL = 8 elements) loads, so a wave streams
// four whole rows per step.  A 16-lane group walks its own keys (group kg of 16 per workgroup,
// keys kg, kg + 16, ...) with a private running softmax for up to 4 query heads of the KV head;
// the groups' partials meet in LDS, the workgroups' (one per context split) in a workspace that
// `sink_attention_merge_kernel` folds together with the sink term and the gate.
// EPL / VPL: elements of a K / V row per lane (D = 16 EPL, E = 16 VPL).
template <typename T, int EPL, int VPL, bool EXT>
__global__ void __launch_bounds__(256)
sink_attention_split_kernel(const T* __restrict__ q, long q_row, long q_head,
                            const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                            const int* __restrict__ block_tables, int max_blocks, int block_size,
                            const int* __restrict__ context_lens, const float* __restrict__ sink,
                            float* __restrict__ ws, float scale, int H, int G, int splits,
                            KeyRule rule) {
    constexpr int D = 16 * EPL, E = 16 * VPL;
    extern __shared__ float sm[];                 // [16 groups][RC][E + 2]
    const int R = H / G, chunks = (R + RC - 1) / RC;
    const int b = blockIdx.x, split = blockIdx.z;
    const int g = blockIdx.y / chunks, h0 = g * R + (blockIdx.y % chunks) * RC;
    const int nr = min(RC, g * R + R - h0);
    const int ctx = context_lens[b];
    const int tid = threadIdx.x, lane16 = tid & 15, kg = tid >> 4;
    const VisibleKeys vis(ctx, rule);
    const int span = ((vis.count + splits - 1) / splits + 15) & ~15;
    const int k_begin = split * span, k_end = min(vis.count, k_begin + span);
    const int* table = block_tables + (long)b * max_blocks;

    float qf[RC][EPL], m[RC], l[RC], acc[RC][VPL], slope[RC];
#pragma unroll
    for (int r = 0; r < RC; ++r) {
        if (r < nr) {
            load_run<T, EPL>(q + b * q_row + (long)(h0 + r) * q_head + lane16 * EPL, qf[r]);
            const float hs = EXT ? rule.head_scale(scale, h0 + r) : scale;
#pragma unroll
            for (int i = 0; i < EPL; ++i) qf[r][i] *= hs;
            m[r] = sink ? sink[h0 + r] : NO_SINK_MAX;
            slope[r] = rule.slopes ? rule.slopes[h0 + r] : 0.f;
        } else {
#pragma unroll
            for (int i = 0; i < EPL; ++i) qf[r][i] = 0.f;
            m[r] = 0.f;
            slope[r] = 0.f;
        }
        l[r] = 0.f;
#pragma unroll
        for (int i = 0; i < VPL; ++i) acc[r][i] = 0.f;
    }
    // two keys per trip: both rows' loads are in flight before the first one is used
    for (int vj = k_begin + kg; vj < k_end; vj += 32) {
        const bool two = vj + 16 < k_end;
        const int j = vis.key(vj), j2 = two ? vis.key(vj + 16) : j;
        const float dist[2] = {(float)(ctx - 1 - j), (float)(ctx - 1 - j2)};
        const long slot = EXT ? vis.row(vj, table, block_size, rule)
                              : (long)table[j / block_size] * block_size + j % block_size;
        const long slot2 = !two ? slot : EXT ? vis.row(vj + 16, table, block_size, rule)
                                             : (long)table[j2 / block_size] * block_size + j2 % block_size;
        float kf[2][EPL], vf[2][VPL];
        load_run<T, EPL>(k_cache + (slot * G + g) * (long)D + lane16 * EPL, kf[0]);
        load_run<T, EPL>(k_cache + (slot2 * G + g) * (long)D + lane16 * EPL, kf[1]);
        load_run<T, VPL>(v_cache + (slot * G + g) * (long)rule.v_stride + lane16 * VPL, vf[0]);
        load_run<T, VPL>(v_cache + (slot2 * G + g) * (long)rule.v_stride + lane16 * VPL, vf[1]);
#pragma unroll
        for (int x = 0; x < 2; ++x) {
            if (x == 1 && !two) break;
#pragma unroll
            for (int r = 0; r < RC; ++r) {
                if (r >= nr) continue;
                float d = 0.f;
#pragma unroll
                for (int i = 0; i < EPL; ++i) d += kf[x][i] * qf[r][i];
                d += __shfl_xor(d, 1, kWave);
                d += __shfl_xor(d, 2, kWave);
                d += __shfl_xor(d, 4, kWave);
                d += __shfl_xor(d, 8, kWave);
                d = (EXT ? rule.capped(d) : d) - slope[r] * dist[x];
                if (d > m[r]) {                    // the running maximum moves: rescale (rare)
                    const float a = expf(m[r] - d);
                    l[r] *= a;
#pragma unroll
                    for (int i = 0; i < VPL; ++i) acc[r][i] *= a;
                    m[r] = d;
                }
                const float p = expf(d - m[r]);
                l[r] += p;
#pragma unroll
                for (int i = 0; i < VPL; ++i) acc[r][i] += p * vf[x][i];
            }
        }
    }
    // the 16 groups' partials -> LDS -> one partial per (head, split)
    constexpr int PS = E + 2;
#pragma unroll
    for (int r = 0; r < RC; ++r) {
        float* dst = sm + (kg * RC + r) * PS;
        if (lane16 == 0) { dst[0] = m[r]; dst[1] = l[r]; }
#pragma unroll
        for (int i = 0; i < VPL; ++i) dst[2 + lane16 * VPL + i] = acc[r][i];
    }
    __syncthreads();
    for (int c = tid; c < nr * PS; c += 256) {
        const int r = c / PS, x = c - r * PS;
        float M = sm[r * PS];
        for (int k = 1; k < 16; ++k) M = fmaxf(M, sm[(k * RC + r) * PS]);
        float v;
        if (x == 0) v = M;
        else {
            v = 0.f;
            for (int k = 0; k < 16; ++k) {
                const float* src = sm + (k * RC + r) * PS;
                v += src[x] * expf(src[0] - M);
            }
        }
        ws[(((long)b * H + h0 + r) * splits + split) * PS + x] = v;
    }
}

template <typename T>
__global__ void sink_attention_merge_kernel(const float* __restrict__ ws,
                                            const float* __restrict__ sink,
                                            const T* __restrict__ gate, long gate_row,
                                            const int* __restrict__ context_lens,
                                            T* __restrict__ out, int H, int E, int splits) {
    const int b = blockIdx.x / H, h = blockIdx.x % H;
    if (context_lens[b] <= 0) return;
    const int PS = E + 2;
    const float* p = ws + ((long)b * H + h) * splits * PS;
    float M = sink ? sink[h] : NO_SINK_MAX;
    for (int s = 0; s < splits; ++s) M = fmaxf(M, p[s * PS]);
    float L = sink ? expf(sink[h] - M) : 0.f;
    for (int s = 0; s < splits; ++s) L += p[s * PS + 1] * expf(p[s * PS] - M);
    float f = 1.f / L;
    if (gate) f *= sigmoidf_(ld(gate + b * gate_row + h));
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        float v = 0.f;
        for (int s = 0; s < splits; ++s) v += p[s * PS + 2 + e] * expf(p[s * PS] - M);
        st(out + ((long)b * H + h) * E + e, v * f);
    }
}

template <typename T, int EPL, int VPL>
static int launch_split(const void* q, long q_row, long q_head, const void* k_cache,
                        const void* v_cache, const void* block_tables, int max_blocks,
                        int block_size, const void* context_lens, const void* sink,
                        const void* gate, long gate_row, void* out, void* ws, float scale, int B,
                        int H, int G, int splits, KeyRule rule, hipStream_t s) {
    constexpr int E = 16 * VPL;
    const int R = H / G, chunks = (R + RC - 1) / RC;
    const size_t lds = 16 * RC * (E + 2) * sizeof(float);
#define SPLIT_LAUNCH(EXT)                                                                         \
    hipLaunchKernelGGL((sink_attention_split_kernel<T, EPL, VPL, EXT>), dim3(B, G * chunks, splits), \
                       dim3(256), lds, s, (const T*)q, q_row, q_head, (const T*)k_cache,          \
                       (const T*)v_cache, (const int*)block_tables, max_blocks, block_size,       \
                       (const int*)context_lens, (const float*)sink, (float*)ws, scale, H, G, splits, \
                       rule)
    if (rule.temps || rule.softcap > 0.f || rule.pool > 0) SPLIT_LAUNCH(true); else SPLIT_LAUNCH(false);
#undef SPLIT_LAUNCH
    if (hipGetLastError() != hipSuccess) return 2;
    hipLaunchKernelGGL(sink_attention_merge_kernel<T>, dim3(B * H), dim3(E >= 128 ? 128 : 64), 0, s,
                       (const float*)ws, (const float*)sink, (const T*)gate, gate_row,
                       (const int*)context_lens, (T*)out, H, E, splits);
    return HYB_LAUNCH_OK();
}

// pooled blocks need a window, no kept first tokens, no distance penalty, and a place in the caches
static bool pool_rule_ok(const KeyRule& r) {
    return r.pool == 0 || (r.pool > 0 && r.window > 0 && r.keep_first == 0 && !r.slopes &&
                           r.pool_rows > 0 && r.pool_base > 0);
}

extern "C" {

// 1 when the split decode kernel has an instance for these head sizes
int hyb_sink_attention_split_ok(int D, int E) {
    return (D == 64 || D == 128 || D == 256) && (E == 64 || E == 128);
}

// Decode rows (row b = sequence b); ws: fp32 workspace of B * H * splits * (E + 2) floats.
int hyb_sink_attention_split(const void* q, long q_row, long q_head, const void* k_cache,
                             const void* v_cache, const void* block_tables, int max_blocks,
                             int block_size, const void* context_lens, const void* sink,
                             const void* gate, long gate_row, void* out, void* ws, float scale,
                             int B, int H, int G, int D, int E, int splits, int window,
                             int keep_first, const void* slopes, int v_stride, const void* temps,
                             float softcap, int pool, int pool_rows, long pool_base, int dt,
                             hipStream_t s) {
    const KeyRule rule{window, keep_first, (const float*)slopes, v_stride > 0 ? v_stride : E,
                       (const float*)temps, softcap, pool, pool_rows, pool_base};
    if (B <= 0) return 0;
    if (!pool_rule_ok(rule)) return 1;
    if (G <= 0 || H % G || splits < 1 || !hyb_sink_attention_split_ok(D, E)) return 1;
    if (rule.v_stride < E || rule.v_stride % 8) return 1;      // 16-byte runs of a value row
    if (((size_t)k_cache | (size_t)v_cache | (size_t)q) % 16 || (q_row * (dt == 0 ? 2 : 4)) % 16) return 1;
#define SPLIT_ARGS q, q_row, q_head, k_cache, v_cache, block_tables, max_blocks, block_size, \
                   context_lens, sink, gate, gate_row, out, ws, scale, B, H, G, splits, rule, s
#define SPLIT_E(T, EPL)                                                  \
    do {                                                                 \
        if (E == 64) return launch_split<T, EPL, 4>(SPLIT_ARGS);         \
        return launch_split<T, EPL, 8>(SPLIT_ARGS);                      \
    } while (0)
#define SPLIT_D(T)                             \
    do {                                       \
        if (D == 64) SPLIT_E(T, 4);            \
        else if (D == 128) SPLIT_E(T, 8);      \
        else SPLIT_E(T, 16);                   \
    } while (0)
    if (dt == 0) SPLIT_D(hyb::bf16_t);
    else if (dt == 2) SPLIT_D(float);
    return 1;
}

// 1 when the tile kernel has an instance for these head sizes (else the row kernel serves)
int hyb_sink_attention_tiles_ok(int D, int E) { return D <= 256 && E <= 256 && !(D > 128 && E > 128); }

// Sequences seq0 .. seq0 + nseq - 1 of a prefill-form step (cu_q / block_tables indexed by the
// absolute sequence number); max_q: longest portion among them.
int hyb_sink_attention_tiles(const void* q, long q_row, long q_head, const void* k_cache,
                             const void* v_cache, const void* block_tables, int max_blocks,
                             int block_size, const void* cu_q, const void* positions,
                             const void* sink, const void* gate, long gate_row, void* out,
                             float scale, int nseq, int seq0, int max_q, int H, int G, int D,
                             int E, int window, int keep_first, const void* slopes, int v_stride,
                             const void* temps, float softcap, int pool, int pool_rows,
                             long pool_base, int dt, hipStream_t s) {
    const KeyRule rule{window, keep_first, (const float*)slopes, v_stride > 0 ? v_stride : E,
                       (const float*)temps, softcap, pool, pool_rows, pool_base};
    if (nseq <= 0 || max_q <= 0) return 0;
    if (!pool_rule_ok(rule)) return 1;
    if (rule.v_stride < E) return 1;
    if (G <= 0 || H % G || !hyb_sink_attention_tiles_ok(D, E)) return 1;
#define TILES_ARGS q, q_row, q_head, k_cache, v_cache, block_tables, max_blocks, block_size, cu_q, \
                   positions, sink, gate, gate_row, out, scale, nseq, seq0, max_q, H, G, D, E
#define TILES_E(T, DP, esz)                                                   \
    do {                                                                      \
        if (E <= 64) return launch_tiles<T, DP, 64>(TILES_ARGS, esz, rule, s);      \
        if (E <= 128) return launch_tiles<T, DP, 128>(TILES_ARGS, esz, rule, s);    \
        if (DP <= 128) return launch_tiles<T, (DP <= 128 ? DP : 64), 256>(TILES_ARGS, esz, rule, s); \
        return 1;                                                             \
    } while (0)
#define TILES_D(T, esz)                                   \
    do {                                                  \
        if (D <= 64) TILES_E(T, 64, esz);                 \
        else if (D <= 128) TILES_E(T, 128, esz);          \
        else TILES_E(T, 256, esz);                        \
    } while (0)
    if (dt == 0) TILES_D(hyb::bf16_t, 2);
    else if (dt == 2) TILES_D(float, 4);
    return 1;
}

// q: [rows, H, D] with strides (q_row, q_head, 1); caches contiguous [blocks, block, G, D|E];
// out contiguous [rows, H, E]; gate [rows, H] with row stride gate_row (or null).
int hyb_sink_attention_rows(const void* q, long q_row, long q_head, const void* k_cache,
                            const void* v_cache, const void* block_tables, int max_blocks,
                            int block_size, const void* row_seq, const void* lens, int len_add,
                            const void* sink, const void* gate, long gate_row, void* out,
                            float scale, long rows, int H, int G, int D, int E, int seq_base,
                            int window, int keep_first, const void* slopes, int v_stride,
                            const void* temps, float softcap, int pool, int pool_rows,
                            long pool_base, int dt, hipStream_t s) {
    const KeyRule rule{window, keep_first, (const float*)slopes, v_stride > 0 ? v_stride : E,
                       (const float*)temps, softcap, pool, pool_rows, pool_base};
    if (rows <= 0) return 0;
    if (!pool_rule_ok(rule)) return 1;
    if (rule.v_stride < E) return 1;
    if (G <= 0 || H % G || E > NACC * TILE || D > 1024) return 1;
    const int fit = NACC * TILE / E;                     // heads whose output columns fit
    const int hpw = fit < RC ? fit : RC;
    const int R = H / G, chunks = (R + hpw - 1) / hpw;
    const size_t lds = (RC * D + RC * TILE + 4 * RC + 3 * RC + 2) * sizeof(float) + TILE * sizeof(long);
    const int esize = dt == 0 ? 2 : 4;
    const int vec_ok = (D % 4 == 0) && (((size_t)k_cache) % 16 == 0) && ((D * esize) % (4 * esize) == 0);
    HYB_DISPATCH(dt, hipLaunchKernelGGL(sink_attention_rows_kernel<T>, dim3(rows, G * chunks),
                                        dim3(TILE), lds, s, (const T*)q, q_row, q_head,
                                        (const T*)k_cache, (const T*)v_cache,
                                        (const int*)block_tables, max_blocks, block_size,
                                        (const int*)row_seq, (const int*)lens, len_add,
                                        (const float*)sink, (const T*)gate, gate_row, (T*)out,
                                        scale, H, G, D, E, vec_ok, seq_base, hpw, rule));
    return HYB_LAUNCH_OK();
}

}  // extern "C"
