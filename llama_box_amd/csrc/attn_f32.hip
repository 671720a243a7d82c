// attn_f32.hip — FLASH_ATTN_EXT in 32-bit arithmetic over a cache read in place (f32, bf16 or f16 rows), for ANY head sizes: the
// query/key size and the value size may differ and need not be 64 or 128.  Scores, soft-max weights and the weighted sum of V are f32
// from start to end (a cache value is widened exactly; nothing is rounded to 16 bits on the way), so an f32 cache gives true 32-bit
// attention.  Optional sinks: one extra score per head that takes part in the soft-max denominator and carries no value (src[4] of the op).
//
// Two kernels:
//   k_attn_f32_rows  — one workgroup per (query token, head), its four waves take the cache in interleaved blocks of 64 cells and merge
//                      their (max, sum, accumulator) through LDS; a block none of whose cells the mask lets through is skipped after
//                      one 128-byte mask read (attention confined to a window or a chunk touches few blocks).  Decode steps and
//                      small batches.
//   k_attn_f32_tile  — prompt batches: a workgroup owns 64 query tokens of one head; K and V blocks of 64 cells are staged through LDS as
//                      f32 once per workgroup and every wave runs 16 of the queries against them (a lane owns one cell for the scores
//                      and one or more value columns for the sum); blocks the mask hides from all 64 queries are skipped.
#include <algorithm>
#include <cstdlib>

#include "dev_util.h"
#include "kernels.h"

namespace mi355x {

template <int T> __device__ __forceinline__ float kv_ld(const char * __restrict__ row, const int i) {
    if constexpr (T == GGML_TYPE_F32) return ((const float *) row)[i];
    else if constexpr (T == GGML_TYPE_BF16) return __uint_as_float((uint32_t) ((const uint16_t *) row)[i] << 16);
    else return h2f(((const uint16_t *) row)[i]);
}

__device__ __forceinline__ float wave_max_f(float v) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_sum_f(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

constexpr int ATTN_F32_MAX_D = 640;   // largest head size (query/key or value): a latent cache row (latent + rotated part) serves as the key of every head
constexpr float ATTN_F32_LOW = -1e30f;  // "no score yet": finite, so that differences of maxima never give NaN

// mask element -> additive term (f16 or f32 mask rows; -inf hides the cell)
__device__ __forceinline__ float mask_ld(const char * __restrict__ mrow, const int mtype, const int64_t j) {
    return mtype == GGML_TYPE_F16 ? h2f(((const uint16_t *) mrow)[j]) : ((const float *) mrow)[j];
}

// the additive term of a visible cell: the mask's value itself, or — with a per-head distance penalty (r1, r2) — the mask's value read as the distance
// between query and cell: -r1 ln(1 + r2 distance)
__device__ __forceinline__ float mask_term(const float mv, const bool pen, const float r1, const float r2) { return pen ? -r1 * logf(1.0f + r2 * mv) : mv; }

// the score of a visible cell before the mask's term: dot product x scale x a per-head factor, then optionally soft-capped (cap tanh(. / cap))
__device__ __forceinline__ float attn_score(const float d, const float scale, const float temp, const float cap) {
    const float sc = d * scale * temp;
    return cap > 0.0f ? cap * tanhf(sc / cap) : sc;
}
// weights that are no soft-max: sigmoid(score + bias) for every visible cell on its own, nothing normalised over the cells (`sig` = per head a factor on the score,
// then per head the bias).  The kernels keep their running maximum at 0, rescale by 1 and skip the division by the sum.
__device__ __forceinline__ float attn_sigmoid(const float z) { return 1.0f / (1.0f + expf(-z)); }

// acc[r] += sum over the block's visible cells of p[cell] * V[cell][lane + 64 r]: no branches around the loads (a lane beyond the row's end re-reads the last
// column, its sum is dropped later; hidden cells enter with weight 0)
template <int VT, int CELLS, int RR>
__device__ __forceinline__ void attn_f32_pv(const float p, const uint64_t live, const char * __restrict__ vbase, const int64_t v_nb1, const int64_t j0, const int64_t n_kv, const int DV,
                                            const int lane, float (&acc)[ATTN_F32_MAX_D / 64]) {
    const uint64_t gmask = CELLS == 64 ? ~0ull : ((1ull << CELLS) - 1ull);
    for (int jj0 = 0; jj0 < 64; jj0 += CELLS) {
        if (!((live >> jj0) & gmask)) continue;
        float vv[CELLS][RR];
#pragma unroll
        for (int u = 0; u < CELLS; ++u) {
            const int64_t cell = j0 + jj0 + u < n_kv ? j0 + jj0 + u : n_kv - 1;
            const char * vrow = vbase + cell * v_nb1;
#pragma unroll
            for (int r = 0; r < RR; ++r) {
                const int dcol = lane + 64 * r;
                vv[u][r] = kv_ld<VT>(vrow, dcol < DV ? dcol : DV - 1);
            }
        }
#pragma unroll
        for (int u = 0; u < CELLS; ++u) {
            const float pj = __shfl(p, jj0 + u, 64);
#pragma unroll
            for (int r = 0; r < RR; ++r) acc[r] = fmaf(pj, vv[u][r], acc[r]);
        }
    }
}

// the same sum for 2-byte value rows of 256 .. 512 entries with a lane owning EIGHT NEIGHBOURING columns (8 lane .. 8 lane + 7): one 16-byte load per cell and lane instead
// of eight 2-byte ones.  Cells enter every column's sum in the same order as above, so the results are the same bit for bit.
template <int VT, int CELLS>
__device__ __forceinline__ void attn_f32_pv8(const float p, const uint64_t live, const char * __restrict__ vbase, const int64_t v_nb1, const int64_t j0, const int64_t n_kv, const int DV,
                                             const int lane, float (&acc)[ATTN_F32_MAX_D / 64]) {
    const uint64_t gmask = (1ull << CELLS) - 1ull;
    const int col = 8 * lane < DV ? 8 * lane : DV - 8;  // (a lane beyond the row's end re-reads the last group; its sums are dropped later)
    for (int jj0 = 0; jj0 < 64; jj0 += CELLS) {
        if (!((live >> jj0) & gmask)) continue;
        uint4 vv[CELLS];
#pragma unroll
        for (int u = 0; u < CELLS; ++u) {
            const int64_t cell = j0 + jj0 + u < n_kv ? j0 + jj0 + u : n_kv - 1;
            vv[u] = *(const uint4 *) (vbase + cell * v_nb1 + col * 2);
        }
#pragma unroll
        for (int u = 0; u < CELLS; ++u) {
            const float pj = __shfl(p, jj0 + u, 64);
            const uint32_t w[4] = {vv[u].x, vv[u].y, vv[u].z, vv[u].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float lo, hi;
                if constexpr (VT == GGML_TYPE_BF16) { lo = __uint_as_float(w[e] << 16); hi = __uint_as_float(w[e] & 0xFFFF0000u); }
                else { lo = h2f((uint16_t) (w[e] & 0xFFFFu)); hi = h2f((uint16_t) (w[e] >> 16)); }
                acc[2 * e] = fmaf(pj, lo, acc[2 * e]);
                acc[2 * e + 1] = fmaf(pj, hi, acc[2 * e + 1]);
            }
        }
    }
}

template <int KT, int VT>
__global__ void __launch_bounds__(256) k_attn_f32_rows(const tdesc q, const tdesc k, const tdesc v, const tdesc mask, const int has_mask, const float * __restrict__ sinks,
                                                       const float * __restrict__ r12, const tdesc dst, const float scale, const float * __restrict__ sig, const float softcap) {
    __shared__ float qs[ATTN_F32_MAX_D];
    __shared__ float part_acc[4][ATTN_F32_MAX_D];
    __shared__ float part_m[4], part_l[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t t = blockIdx.x, h = blockIdx.y;
    const int DK = (int) q.ne[0], DV = (int) v.ne[0];
    const int64_t n_kv = k.ne[1];
    const int64_t g = h / (q.ne[2] / k.ne[2]);
    const char * qrow = q.data + t * q.nb[1] + h * q.nb[2];
    for (int i = threadIdx.x; i < DK; i += 256) qs[i] = ((const float *) qrow)[i];
    __syncthreads();
    const char * mrow = has_mask ? mask.data + t * mask.nb[1] : nullptr;
    const char * kbase = k.data + g * k.nb[2];
    const char * vbase = v.data + g * v.nb[2];
    const bool pen = r12 != nullptr;
    const float r1 = pen ? r12[h] : 0.0f, r2 = pen ? r12[q.ne[2] + h] : 0.0f;
    // (value rows of 256 .. 512 two-byte entries: a lane owns eight neighbouring columns)
    const bool v_vec8 = VT != GGML_TYPE_F32 && DV > 256 && DV <= 512 && (DV % 8) == 0 && (v.nb[1] % 16) == 0 && (v.nb[2] % 16) == 0 && (((uintptr_t) v.data) & 15) == 0;
    const bool k_vec = KT != GGML_TYPE_F32 && (DK % 8) == 0 && (k.nb[1] % 16) == 0 && (k.nb[2] % 16) == 0 && (((uintptr_t) k.data) & 15) == 0;
    const bool sgm = sig != nullptr;
    const float s_temp = sgm ? sig[h] : 1.0f, s_bias = sgm ? sig[q.ne[2] + h] : 0.0f;
    float m = sgm ? 0.0f : ATTN_F32_LOW, l = 0.0f;
    if (sinks && wave == 0 && !sgm) { m = sinks[h]; l = 1.0f; }  // the sink: exp(sink - m) = 1 in the denominator, nothing in the numerator
    float acc[ATTN_F32_MAX_D / 64];
#pragma unroll
    for (int r = 0; r < ATTN_F32_MAX_D / 64; ++r) acc[r] = 0.0f;
    for (int64_t j0 = (int64_t) wave * 64; j0 < n_kv; j0 += 256) {
        const int64_t j = j0 + lane;
        float mv = -INFINITY;
        if (j < n_kv) mv = has_mask ? mask_ld(mrow, mask.type, j) : 0.0f;
        const bool vis = mv > -INFINITY;
        const uint64_t live = __ballot(vis);
        if (!live) continue;
        float s = -INFINITY;
        if (vis) {
            const char * krow = kbase + j * k.nb[1];
            float d = 0.0f;
            if constexpr (KT != GGML_TYPE_F32) {
                if (k_vec) {  // 16-byte loads of eight 2-byte values; the sum runs over i in the same order as the scalar loop below
                    for (int i = 0; i < DK; i += 8) {
                        const uint4 w = *(const uint4 *) (krow + i * 2);
                        const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            float lo, hi;
                            if constexpr (KT == GGML_TYPE_BF16) { lo = __uint_as_float(u[e] << 16); hi = __uint_as_float(u[e] & 0xFFFF0000u); }
                            else { lo = h2f((uint16_t) (u[e] & 0xFFFFu)); hi = h2f((uint16_t) (u[e] >> 16)); }
                            d = fmaf(qs[i + 2 * e], lo, d);
                            d = fmaf(qs[i + 2 * e + 1], hi, d);
                        }
                    }
                } else
                for (int i = 0; i < DK; ++i) d = fmaf(qs[i], kv_ld<KT>(krow, i), d);
            } else
            for (int i = 0; i < DK; ++i) d = fmaf(qs[i], kv_ld<KT>(krow, i), d);
            s = attn_score(d, scale, s_temp, softcap) + mask_term(mv, pen, r1, r2);
        }
        float p, corr;
        if (sgm) {
            p = vis ? attn_sigmoid(s + s_bias) : 0.0f;
            corr = 1.0f;
        } else {
            const float m_new = fmaxf(m, wave_max_f(s));
            p = vis ? expf(s - m_new) : 0.0f;
            corr = expf(m - m_new);
            l = l * corr + wave_sum_f(p);
            m = m_new;
        }
#pragma unroll
        for (int r = 0; r < ATTN_F32_MAX_D / 64; ++r) acc[r] *= corr;
        // the visible cells' value rows, CELLS at a time with all their loads in flight together: a wave pays one trip to memory per group (measured: 2 us
        // on an otherwise idle chip), so the groups are as large as the registers allow — 32 cells for value sizes up to 128, 16 beyond
        if constexpr (VT != GGML_TYPE_F32) {
            if (v_vec8) { attn_f32_pv8<VT, 16>(p, live, vbase, v.nb[1], j0, n_kv, DV, lane, acc); continue; }
        }
        if (DV <= 128) attn_f32_pv<VT, 32, 2>(p, live, vbase, v.nb[1], j0, n_kv, DV, lane, acc);
        else if (DV <= 256) attn_f32_pv<VT, 16, 4>(p, live, vbase, v.nb[1], j0, n_kv, DV, lane, acc);
        else attn_f32_pv<VT, 8, ATTN_F32_MAX_D / 64>(p, live, vbase, v.nb[1], j0, n_kv, DV, lane, acc);
    }
    if (lane == 0) { part_m[wave] = m; part_l[wave] = l; }
    if (v_vec8) {
#pragma unroll
        for (int e = 0; e < 8; ++e) if (8 * lane + e < DV) part_acc[wave][8 * lane + e] = acc[e];
    } else {
#pragma unroll
        for (int r = 0; r < ATTN_F32_MAX_D / 64; ++r) {
            const int dcol = lane + 64 * r;
            if (dcol < DV) part_acc[wave][dcol] = acc[r];
        }
    }
    __syncthreads();
    if (wave != 0) return;
    float M = part_m[0];
    for (int w = 1; w < 4; ++w) M = fmaxf(M, part_m[w]);
    float L = 0.0f, cw[4];
    for (int w = 0; w < 4; ++w) { cw[w] = expf(part_m[w] - M); L += part_l[w] * cw[w]; }
    const float inv = sgm ? 1.0f : (L > 0.0f ? 1.0f / L : 0.0f);
    float * out = (float *) (dst.data + h * dst.nb[1] + t * dst.nb[2]);
    for (int dcol = lane; dcol < DV; dcol += 64) {
        float o = 0.0f;
        for (int w = 0; w < 4; ++w) o += part_acc[w][dcol] * cw[w];
        out[dcol] = o * inv;
    }
}

// prompt batches: 64 query tokens x one head per workgroup; K / V blocks of 64 cells staged in LDS as f32
template <int KT, int VT, int DKP, int DVP>   // DKP / DVP: head sizes rounded up to a multiple of 32 / 64 (LDS row lengths)
__global__ void __launch_bounds__(256) k_attn_f32_tile(const tdesc q, const tdesc k, const tdesc v, const tdesc mask, const float * __restrict__ sinks,
                                                       const float * __restrict__ r12, const tdesc dst, const float scale, const float * __restrict__ sig, const float softcap) {
    constexpr int QT = 64, KB = 64, QW = QT / 4;  // queries per workgroup, cells per block, queries per wave
    constexpr int KS = DKP + 1;                   // K row stride in LDS (odd: lanes that read column i of 64 different rows hit 64 different banks)
    extern __shared__ float lds[];
    float * Ks = lds;                    // [KB][KS]
    float * Vs = Ks + KB * KS;           // [KB][DVP]
    float * Qs = Vs + KB * DVP;          // [QT][DKP]
    __shared__ int blk_live;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t t0 = (int64_t) blockIdx.x * QT, h = blockIdx.y;
    const int DK = (int) q.ne[0], DV = (int) v.ne[0];
    const int64_t n_kv = k.ne[1], n_q = q.ne[1];
    const int64_t g = h / (q.ne[2] / k.ne[2]);
    const char * kbase = k.data + g * k.nb[2];
    const char * vbase = v.data + g * v.nb[2];
    const bool pen = r12 != nullptr;
    const float r1 = pen ? r12[h] : 0.0f, r2 = pen ? r12[q.ne[2] + h] : 0.0f;
    for (int e = threadIdx.x; e < QT * DKP; e += 256) {
        const int qi = e / DKP, i = e % DKP;
        const int64_t t = t0 + qi;
        Qs[e] = (t < n_q && i < DK) ? ((const float *) (q.data + t * q.nb[1] + h * q.nb[2]))[i] : 0.0f;
    }
    const bool sgm = sig != nullptr;
    const float s_temp = sgm ? sig[h] : 1.0f, s_bias = sgm ? sig[q.ne[2] + h] : 0.0f;
    float m[QW], l[QW], acc[QW][DVP / 64];
#pragma unroll
    for (int qi = 0; qi < QW; ++qi) {
        m[qi] = sgm ? 0.0f : (sinks ? sinks[h] : ATTN_F32_LOW);
        l[qi] = (sinks && !sgm) ? 1.0f : 0.0f;
#pragma unroll
        for (int r = 0; r < DVP / 64; ++r) acc[qi][r] = 0.0f;
    }
    for (int64_t j0 = 0; j0 < n_kv; j0 += KB) {
        // does any of the 64 queries see any of the 64 cells?  (one mask element per thread and query row quarter)
        __syncthreads();
        if (threadIdx.x == 0) blk_live = 0;
        __syncthreads();
        {
            bool any = false;
            for (int qi = wave; qi < QT; qi += 4) {
                const int64_t t = t0 + qi, j = j0 + lane;
                if (t < n_q && j < n_kv) any = any || mask_ld(mask.data + t * mask.nb[1], mask.type, j) > -INFINITY;
            }
            if (__ballot(any) && lane == 0) blk_live = 1;
        }
        __syncthreads();
        if (!blk_live) continue;
        for (int e = threadIdx.x; e < KB * DKP; e += 256) {
            const int r = e / DKP, i = e % DKP;
            const int64_t j = j0 + r;
            Ks[r * KS + i] = (j < n_kv && i < DK) ? kv_ld<KT>(kbase + j * k.nb[1], i) : 0.0f;
        }
        for (int e = threadIdx.x; e < KB * DVP; e += 256) {
            const int r = e / DVP, i = e % DVP;
            const int64_t j = j0 + r;
            Vs[e] = (j < n_kv && i < DV) ? kv_ld<VT>(vbase + j * v.nb[1], i) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int qi = 0; qi < QW; ++qi) {
            const int ql = wave * QW + qi;
            const int64_t t = t0 + ql, j = j0 + lane;
            float mv = -INFINITY;
            if (t < n_q && j < n_kv) mv = mask_ld(mask.data + t * mask.nb[1], mask.type, j);
            const bool vis = mv > -INFINITY;
            const uint64_t live = __ballot(vis);
            if (!live) continue;
            float d = 0.0f;
            const float * qr = Qs + ql * DKP;
            const float * kr = Ks + lane * KS;
            for (int i = 0; i < DK; ++i) d = fmaf(qr[i], kr[i], d);
            const float s = vis ? attn_score(d, scale, s_temp, softcap) + mask_term(mv, pen, r1, r2) : -INFINITY;
            float p, corr;
            if (sgm) {
                p = vis ? attn_sigmoid(s + s_bias) : 0.0f;
                corr = 1.0f;
            } else {
                const float m_new = fmaxf(m[qi], wave_max_f(s));
                p = vis ? expf(s - m_new) : 0.0f;
                corr = expf(m[qi] - m_new);
                l[qi] = l[qi] * corr + wave_sum_f(p);
                m[qi] = m_new;
            }
#pragma unroll
            for (int r = 0; r < DVP / 64; ++r) acc[qi][r] *= corr;
            uint64_t todo = live;
            while (todo) {
                const int jj = __builtin_ctzll(todo);
                todo &= todo - 1;
                const float pj = __shfl(p, jj, 64);
#pragma unroll
                for (int r = 0; r < DVP / 64; ++r) acc[qi][r] = fmaf(pj, Vs[jj * DVP + lane + 64 * r], acc[qi][r]);
            }
        }
    }
#pragma unroll
    for (int qi = 0; qi < QW; ++qi) {
        const int64_t t = t0 + wave * QW + qi;
        if (t >= n_q) continue;
        const float inv = sgm ? 1.0f : (l[qi] > 0.0f ? 1.0f / l[qi] : 0.0f);
        float * out = (float *) (dst.data + h * dst.nb[1] + t * dst.nb[2]);
#pragma unroll
        for (int r = 0; r < DVP / 64; ++r) {
            const int dcol = lane + 64 * r;
            if (dcol < DV) out[dcol] = acc[qi][r] * inv;
        }
    }
}

// ------------------------------------------------------------------------------------------------ prompt batches over a bf16 cache: the matrix cores
// k_attn_mma_bf16: a wave owns 32 query tokens of one head; a workgroup is 1, 2 or 4 such waves sharing the staged V^T block.  Per block of 32 cells
//   S^T = K . Q^T   on v_mfma_f32_32x32x16_bf16 (first operand: the cells' bf16 rows straight from the cache, 16 bytes a lane; second: the wave's queries,
//                   rounded to bf16 once and kept in registers) — a lane then holds 16 scores of ITS query (its half-wave's cells), so the running maximum,
//                   the sum and the rescaling are per-lane scalars and one exchange with the other half-wave;
//   scores, maxima, exponentials and sums are f32;
//   O^T += V^T . P^T  on the same instruction, V^T staged through LDS (bf16, transposed on the way in), the weights P given as TWO bf16 terms
//                   (p = hi + lo, |lo| <= 2^-9 |p|): the f32 weights enter the sum to 2^-17, not rounded to 8 bits.
// The key order inside the second product is the order the first product's registers come in (both operands permuted alike).
// Blocks that the mask hides from all of a workgroup's queries are skipped after the mask read.  Head sizes: multiples of 8 up to 16 DK16 / 32 DVT.
typedef __bf16 att_bf8 __attribute__((ext_vector_type(8)));
typedef float att_f16v __attribute__((ext_vector_type(16)));
__device__ __forceinline__ uint32_t att_bf16_bits(const float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
template <int DK16, int DVT>
__global__ void __launch_bounds__(256) k_attn_mma_bf16(const tdesc q, const tdesc k, const tdesc v, const tdesc mask, const float * __restrict__ sinks, const float * __restrict__ r12, const tdesc dst,
                                                       const float scale, const float * __restrict__ sig, const float softcap) {
    constexpr int VS = 36;  // V^T row stride in LDS (bf16 elements): 72 bytes keeps the 8-byte reads aligned and spreads the rows over the banks
    __shared__ __attribute__((aligned(16))) uint16_t Vt[DVT * 32 * VS];
    __shared__ int flag[2];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 31, g = lane >> 5;
    const int64_t h = blockIdx.y, n_q = q.ne[1], n_kv = k.ne[1];
    const int DK = (int) q.ne[0], DV = (int) v.ne[0];
    const int64_t tq = (int64_t) blockIdx.x * (blockDim.x / 2) + wave * 32 + n;  // this lane's query (a workgroup of 1, 2 or 4 waves: 32 queries a wave)
    const bool q_live = tq < n_q;
    const int64_t kvh = h / (q.ne[2] / k.ne[2]);
    const char * kbase = k.data + kvh * k.nb[2];
    const char * vbase = v.data + kvh * v.nb[2];
    // the wave's queries as second operands: element group (16 s + 8 g .. + 7) of query n
    uint4 qf[DK16];
    {
        const float * qrow = (const float *) (q.data + (q_live ? tq : 0) * q.nb[1] + h * q.nb[2]);
#pragma unroll
        for (int s = 0; s < DK16; ++s) {
            const int i0 = 16 * s + 8 * g;
            uint32_t b[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) b[e] = (q_live && i0 + e < DK) ? att_bf16_bits(qrow[i0 + e]) : 0u;
            qf[s] = make_uint4(b[0] | (b[1] << 16), b[2] | (b[3] << 16), b[4] | (b[5] << 16), b[6] | (b[7] << 16));
        }
    }
    const bool pen = r12 != nullptr;
    const float r1 = pen ? r12[h] : 0.0f, r2 = pen ? r12[q.ne[2] + h] : 0.0f;
    const bool sgm = sig != nullptr;
    const float s_temp = sgm ? sig[h] : 1.0f, s_bias = sgm ? sig[q.ne[2] + h] : 0.0f;
    float m = sgm ? 0.0f : (sinks ? sinks[h] : ATTN_F32_LOW), l = (sinks && !sgm) ? 1.0f : 0.0f;
    att_f16v O[DVT];
#pragma unroll
    for (int dt = 0; dt < DVT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) O[dt][i] = 0.0f;
    const char * mrow = mask.data + (q_live ? tq : 0) * mask.nb[1];
    if (threadIdx.x < 2) flag[threadIdx.x] = 0;
    __syncthreads();
    // this lane's 16 mask terms of a block: cells j0 + 8 b + 4 g .. + 3, b = 0 .. 3 (register i = 4 b + r); the NEXT block's terms are requested while the
    // current block is worked on (three dependent trips to memory per block — mask, V, K — were what bound this kernel)
    auto load_mask = [&](const int64_t j0, float (&mv)[16]) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int64_t j = j0 + 8 * b + 4 * g;
            float4 t = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
            if (q_live && j + 3 < n_kv) t = *(const float4 *) (mrow + j * 4);
            else if (q_live) {
                if (j < n_kv) t.x = ((const float *) mrow)[j];
                if (j + 1 < n_kv) t.y = ((const float *) mrow)[j + 1];
                if (j + 2 < n_kv) t.z = ((const float *) mrow)[j + 2];
            }
            mv[4 * b] = t.x; mv[4 * b + 1] = t.y; mv[4 * b + 2] = t.z; mv[4 * b + 3] = t.w;
        }
    };
    float mv_next[16];
    load_mask(0, mv_next);
    for (int64_t j0 = 0, blk = 0; j0 < n_kv; j0 += 32, ++blk) {
        float mv[16];
        bool any = false;
#pragma unroll
        for (int i = 0; i < 16; ++i) { mv[i] = mv_next[i]; any = any || mv[i] > -INFINITY; }
        if (j0 + 32 < n_kv) load_mask(j0 + 32, mv_next);
        const bool wave_any = __ballot(any) != 0;
        if (threadIdx.x == 0) flag[(blk + 1) & 1] = 0;
        if (wave_any && lane == 0) flag[blk & 1] = 1;
        __syncthreads();
        if (!flag[blk & 1]) continue;  // (the same answer for every thread of the workgroup)
        // the block's K operands are requested first, so that they travel while V^T is staged
        uint4 kf[DK16];
        {
            const int64_t cell = j0 + n < n_kv ? j0 + n : n_kv - 1;
            const char * krow = kbase + cell * k.nb[1] + g * 16;
#pragma unroll
            for (int s = 0; s < DK16; ++s) {
                kf[s] = make_uint4(0, 0, 0, 0);
                if (wave_any && 16 * s + 8 * g < DK) kf[s] = *(const uint4 *) (krow + s * 32);
            }
        }
        // V^T of the block into LDS: a thread takes 8 consecutive value entries of FOUR neighbouring cells and writes eight 8-byte groups (4 cells of one entry)
        for (int e0 = threadIdx.x; e0 < 8 * (DVT * 4); e0 += blockDim.x) {
            const int cg = e0 / (DVT * 4), c8 = e0 % (DVT * 4);
            uint32_t u[4][4];
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) {
                uint4 t = make_uint4(0, 0, 0, 0);
                if (j0 + 4 * cg + cc < n_kv && 8 * c8 < DV) t = *(const uint4 *) (vbase + (j0 + 4 * cg + cc) * v.nb[1] + c8 * 16);
                u[cc][0] = t.x; u[cc][1] = t.y; u[cc][2] = t.z; u[cc][3] = t.w;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // entries 2 e (low halves) and 2 e + 1 (high halves) of the four cells
                const uint2 lo2 = make_uint2((u[0][e] & 0xFFFFu) | (u[1][e] << 16), (u[2][e] & 0xFFFFu) | (u[3][e] << 16));
                const uint2 hi2 = make_uint2((u[0][e] >> 16) | (u[1][e] & 0xFFFF0000u), (u[2][e] >> 16) | (u[3][e] & 0xFFFF0000u));
                *(uint2 *) (Vt + (8 * c8 + 2 * e) * VS + 4 * cg) = lo2;
                *(uint2 *) (Vt + (8 * c8 + 2 * e + 1) * VS + 4 * cg) = hi2;
            }
        }
        __syncthreads();
        if (!wave_any) continue;  // (wave-uniform; no barrier follows inside this iteration)
        att_f16v S;
#pragma unroll
        for (int i = 0; i < 16; ++i) S[i] = 0.0f;
#pragma unroll
        for (int s = 0; s < DK16; ++s) S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(att_bf8, kf[s]), __builtin_bit_cast(att_bf8, qf[s]), S, 0, 0, 0);
        float mx = ATTN_F32_LOW;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            S[i] = mv[i] > -INFINITY ? attn_score(S[i], scale, s_temp, softcap) + mask_term(mv[i], pen, r1, r2) : -INFINITY;
            mx = fmaxf(mx, S[i]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = sgm ? 0.0f : fmaxf(m, mx);
        const float corr = sgm ? 1.0f : expf(m - m_new);
        float ps = 0.0f;
        uint32_t hi[8], lo[8];
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
            const float p0 = sgm ? (S[i] > -INFINITY ? attn_sigmoid(S[i] + s_bias) : 0.0f) : expf(S[i] - m_new);
            const float p1 = sgm ? (S[i + 1] > -INFINITY ? attn_sigmoid(S[i + 1] + s_bias) : 0.0f) : expf(S[i + 1] - m_new);
            ps += p0 + p1;
            const uint32_t h0 = att_bf16_bits(p0), h1 = att_bf16_bits(p1);
            hi[i >> 1] = h0 | (h1 << 16);
            lo[i >> 1] = att_bf16_bits(p0 - __uint_as_float(h0 << 16)) | (att_bf16_bits(p1 - __uint_as_float(h1 << 16)) << 16);
        }
        ps += __shfl_xor(ps, 32, 64);
        l = l * corr + ps;
        m = m_new;
#pragma unroll
        for (int dt = 0; dt < DVT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) O[dt][i] *= corr;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            const uint4 ph = make_uint4(hi[4 * s2], hi[4 * s2 + 1], hi[4 * s2 + 2], hi[4 * s2 + 3]);
            const uint4 pl = make_uint4(lo[4 * s2], lo[4 * s2 + 1], lo[4 * s2 + 2], lo[4 * s2 + 3]);
#pragma unroll
            for (int dt = 0; dt < DVT; ++dt) {
                const uint16_t * vr = Vt + (32 * dt + n) * VS + 16 * s2 + 4 * g;
                const uint2 a0 = *(const uint2 *) vr, a1 = *(const uint2 *) (vr + 8);
                const uint4 vf = make_uint4(a0.x, a0.y, a1.x, a1.y);
                O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(att_bf8, vf), __builtin_bit_cast(att_bf8, ph), O[dt], 0, 0, 0);
                O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(att_bf8, vf), __builtin_bit_cast(att_bf8, pl), O[dt], 0, 0, 0);
            }
        }
    }
    if (!q_live) return;
    const float inv = sgm ? 1.0f : (l > 0.0f ? 1.0f / l : 0.0f);
    float * out = (float *) (dst.data + h * dst.nb[1] + tq * dst.nb[2]);
#pragma unroll
    for (int dt = 0; dt < DVT; ++dt)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int d0 = 32 * dt + 8 * b + 4 * g;
            if (d0 + 3 < DV) *(float4 *) (out + d0) = make_float4(O[dt][4 * b] * inv, O[dt][4 * b + 1] * inv, O[dt][4 * b + 2] * inv, O[dt][4 * b + 3] * inv);
            else
                for (int r = 0; r < 4; ++r) if (d0 + r < DV) out[d0 + r] = O[dt][4 * b + r] * inv;
        }
}
// k_attn_mma_bf16_wide: the same scheme for ONE key/value head shared by all query heads and rows wider than a wave can hold — a latent cache row [latent | rotated part] of
// several hundred values, its leading part the value.  The queries of a workgroup are 32 (token, head) pairs (head fastest); its four waves share them: wave w computes the
// partial scores over a quarter of the key entries, the partials meet in LDS (every wave adds them in the order 0 .. 3 and so holds the same scores), every wave runs the f32
// soft-max, and wave w accumulates a quarter of the value entries (O^T tiles of 32).  V^T of the block is staged once for all four.  DKQ: 16-entry key groups per wave, DVQ:
// 32-entry value tiles per wave.
template <int DKQ, int DVQ>
__global__ void __launch_bounds__(256) k_attn_mma_bf16_wide(const tdesc q, const tdesc k, const tdesc v, const tdesc mask, const float * __restrict__ sinks, const float * __restrict__ r12,
                                                            const tdesc dst, const float scale, const float * __restrict__ sig, const float softcap) {
    constexpr int VS = 36;
    constexpr int DVT = 4 * DVQ;
    __shared__ __attribute__((aligned(16))) uint16_t Vt[DVT * 32 * VS];
    __shared__ float Sp[4][16][64];
    __shared__ int flag[2];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 31, g = lane >> 5;
    const int64_t H = q.ne[2], n_tok = q.ne[1], n_kv = k.ne[1];
    const int DK = (int) q.ne[0], DV = (int) v.ne[0];
    const int64_t qi = (int64_t) blockIdx.x * 32 + n;  // this lane's (token, head) pair
    const bool q_live = qi < n_tok * H;
    const int64_t tq = q_live ? qi / H : 0, h = q_live ? qi % H : 0;
    const char * kbase = k.data;
    const char * vbase = v.data;
    uint4 qf[DKQ];
    {
        const float * qrow = (const float *) (q.data + tq * q.nb[1] + h * q.nb[2]);
#pragma unroll
        for (int s = 0; s < DKQ; ++s) {
            const int i0 = 16 * (wave * DKQ + s) + 8 * g;
            uint32_t b[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) b[e] = (q_live && i0 + e < DK) ? att_bf16_bits(qrow[i0 + e]) : 0u;
            qf[s] = make_uint4(b[0] | (b[1] << 16), b[2] | (b[3] << 16), b[4] | (b[5] << 16), b[6] | (b[7] << 16));
        }
    }
    const bool pen = r12 != nullptr;
    const float r1 = pen ? r12[h] : 0.0f, r2 = pen ? r12[H + h] : 0.0f;
    const bool sgm = sig != nullptr;
    const float s_temp = sgm ? sig[h] : 1.0f, s_bias = sgm ? sig[q.ne[2] + h] : 0.0f;
    float m = sgm ? 0.0f : (sinks ? sinks[h] : ATTN_F32_LOW), l = (sinks && !sgm) ? 1.0f : 0.0f;
    att_f16v O[DVQ];
#pragma unroll
    for (int dt = 0; dt < DVQ; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) O[dt][i] = 0.0f;
    const char * mrow = mask.data + tq * mask.nb[1];
    if (threadIdx.x < 2) flag[threadIdx.x] = 0;
    __syncthreads();
    auto load_mask = [&](const int64_t j0, float (&mv)[16]) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int64_t j = j0 + 8 * b + 4 * g;
            float4 t = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
            if (q_live && j + 3 < n_kv) t = *(const float4 *) (mrow + j * 4);
            else if (q_live) {
                if (j < n_kv) t.x = ((const float *) mrow)[j];
                if (j + 1 < n_kv) t.y = ((const float *) mrow)[j + 1];
                if (j + 2 < n_kv) t.z = ((const float *) mrow)[j + 2];
            }
            mv[4 * b] = t.x; mv[4 * b + 1] = t.y; mv[4 * b + 2] = t.z; mv[4 * b + 3] = t.w;
        }
    };
    float mv_next[16];
    load_mask(0, mv_next);
    for (int64_t j0 = 0, blk = 0; j0 < n_kv; j0 += 32, ++blk) {
        float mv[16];
        bool any = false;
#pragma unroll
        for (int i = 0; i < 16; ++i) { mv[i] = mv_next[i]; any = any || mv[i] > -INFINITY; }
        if (j0 + 32 < n_kv) load_mask(j0 + 32, mv_next);
        const bool wave_any = __ballot(any) != 0;  // (the four waves hold the same queries: the same answer in each)
        if (threadIdx.x == 0) flag[(blk + 1) & 1] = 0;
        if (wave_any && lane == 0) flag[blk & 1] = 1;
        __syncthreads();
        if (!flag[blk & 1]) continue;
        // this wave's quarter of the block's key entries, straight from the cache rows
        uint4 kf[DKQ];
        {
            const int64_t cell = j0 + n < n_kv ? j0 + n : n_kv - 1;
            const char * krow = kbase + cell * k.nb[1] + g * 16;
#pragma unroll
            for (int s = 0; s < DKQ; ++s) {
                const int sg = wave * DKQ + s;
                kf[s] = make_uint4(0, 0, 0, 0);
                if (16 * sg + 8 * g < DK) kf[s] = *(const uint4 *) (krow + sg * 32);
            }
        }
        // V^T of the block (all value entries) into LDS, as in k_attn_mma_bf16
        for (int e0 = threadIdx.x; e0 < 8 * (DVT * 4); e0 += 256) {
            const int cg = e0 / (DVT * 4), c8 = e0 % (DVT * 4);
            uint32_t u[4][4];
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) {
                uint4 t = make_uint4(0, 0, 0, 0);
                if (j0 + 4 * cg + cc < n_kv && 8 * c8 < DV) t = *(const uint4 *) (vbase + (j0 + 4 * cg + cc) * v.nb[1] + c8 * 16);
                u[cc][0] = t.x; u[cc][1] = t.y; u[cc][2] = t.z; u[cc][3] = t.w;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint2 lo2 = make_uint2((u[0][e] & 0xFFFFu) | (u[1][e] << 16), (u[2][e] & 0xFFFFu) | (u[3][e] << 16));
                const uint2 hi2 = make_uint2((u[0][e] >> 16) | (u[1][e] & 0xFFFF0000u), (u[2][e] >> 16) | (u[3][e] & 0xFFFF0000u));
                *(uint2 *) (Vt + (8 * c8 + 2 * e) * VS + 4 * cg) = lo2;
                *(uint2 *) (Vt + (8 * c8 + 2 * e + 1) * VS + 4 * cg) = hi2;
            }
        }
        // partial scores over this wave's key entries
        {
            att_f16v Sw;
#pragma unroll
            for (int i = 0; i < 16; ++i) Sw[i] = 0.0f;
#pragma unroll
            for (int s = 0; s < DKQ; ++s) Sw = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(att_bf8, kf[s]), __builtin_bit_cast(att_bf8, qf[s]), Sw, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 16; ++i) Sp[wave][i][lane] = Sw[i];
        }
        __syncthreads();
        att_f16v S;
#pragma unroll
        for (int i = 0; i < 16; ++i) S[i] = ((Sp[0][i][lane] + Sp[1][i][lane]) + Sp[2][i][lane]) + Sp[3][i][lane];
        float mx = ATTN_F32_LOW;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            S[i] = mv[i] > -INFINITY ? attn_score(S[i], scale, s_temp, softcap) + mask_term(mv[i], pen, r1, r2) : -INFINITY;
            mx = fmaxf(mx, S[i]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = sgm ? 0.0f : fmaxf(m, mx);
        const float corr = sgm ? 1.0f : expf(m - m_new);
        float ps = 0.0f;
        uint32_t hi[8], lo[8];
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
            const float p0 = sgm ? (S[i] > -INFINITY ? attn_sigmoid(S[i] + s_bias) : 0.0f) : expf(S[i] - m_new);
            const float p1 = sgm ? (S[i + 1] > -INFINITY ? attn_sigmoid(S[i + 1] + s_bias) : 0.0f) : expf(S[i + 1] - m_new);
            ps += p0 + p1;
            const uint32_t h0 = att_bf16_bits(p0), h1 = att_bf16_bits(p1);
            hi[i >> 1] = h0 | (h1 << 16);
            lo[i >> 1] = att_bf16_bits(p0 - __uint_as_float(h0 << 16)) | (att_bf16_bits(p1 - __uint_as_float(h1 << 16)) << 16);
        }
        ps += __shfl_xor(ps, 32, 64);
        l = l * corr + ps;
        m = m_new;
#pragma unroll
        for (int dt = 0; dt < DVQ; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) O[dt][i] *= corr;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            const uint4 ph = make_uint4(hi[4 * s2], hi[4 * s2 + 1], hi[4 * s2 + 2], hi[4 * s2 + 3]);
            const uint4 pl = make_uint4(lo[4 * s2], lo[4 * s2 + 1], lo[4 * s2 + 2], lo[4 * s2 + 3]);
#pragma unroll
            for (int dt = 0; dt < DVQ; ++dt) {
                const uint16_t * vr = Vt + (32 * (wave * DVQ + dt) + n) * VS + 16 * s2 + 4 * g;
                const uint2 a0 = *(const uint2 *) vr, a1 = *(const uint2 *) (vr + 8);
                const uint4 vf = make_uint4(a0.x, a0.y, a1.x, a1.y);
                O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(att_bf8, vf), __builtin_bit_cast(att_bf8, ph), O[dt], 0, 0, 0);
                O[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(att_bf8, vf), __builtin_bit_cast(att_bf8, pl), O[dt], 0, 0, 0);
            }
        }
    }
    if (!q_live) return;
    const float inv = sgm ? 1.0f : (l > 0.0f ? 1.0f / l : 0.0f);
    float * out = (float *) (dst.data + h * dst.nb[1] + tq * dst.nb[2]);
#pragma unroll
    for (int dt = 0; dt < DVQ; ++dt)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int d0 = 32 * (wave * DVQ + dt) + 8 * b + 4 * g;
            if (d0 + 3 < DV) *(float4 *) (out + d0) = make_float4(O[dt][4 * b] * inv, O[dt][4 * b + 1] * inv, O[dt][4 * b + 2] * inv, O[dt][4 * b + 3] * inv);
            else
                for (int r = 0; r < 4; ++r) if (d0 + r < DV) out[d0 + r] = O[dt][4 * b + r] * inv;
        }
}
// one key/value head, rows beyond what k_attn_mma_bf16 holds (up to 640 key and 512 value entries), at least 128 (token, head) pairs: a workgroup walks the whole cache for 32
// pairs, so a decode step's few pairs are better served by the row kernel's workgroup per pair
static bool attn_mma_bf16_wide_ok(const tdesc & q, const tdesc & k, const tdesc & v, const tdesc * mask, const tdesc & dst) {
    if (!mask || mask->type != GGML_TYPE_F32 || (mask->nb[1] % 16) != 0 || (((uintptr_t) mask->data) & 15)) return false;
    if (k.type != GGML_TYPE_BF16 || v.type != GGML_TYPE_BF16 || k.ne[2] != 1 || q.ne[1] * q.ne[2] < 128) return false;
    if ((q.ne[0] % 8) != 0 || (v.ne[0] % 8) != 0 || (q.ne[0] <= 128 && v.ne[0] <= 128) || q.ne[0] > 640 || v.ne[0] > 512) return false;
    if ((k.nb[1] % 16) || (v.nb[1] % 16) || (((uintptr_t) k.data | (uintptr_t) v.data | (uintptr_t) dst.data) & 15)) return false;
    if ((dst.nb[1] % 16) || (dst.nb[2] % 16)) return false;
    return true;
}

static bool attn_mma_bf16_ok(const tdesc & q, const tdesc & k, const tdesc & v, const tdesc * mask, const tdesc & dst) {
    if (!mask || mask->type != GGML_TYPE_F32 || (mask->nb[1] % 16) != 0 || (((uintptr_t) mask->data) & 15)) return false;
    if (k.type != GGML_TYPE_BF16 || v.type != GGML_TYPE_BF16 || q.ne[1] < 32) return false;
    if ((q.ne[0] % 8) != 0 || (v.ne[0] % 8) != 0 || q.ne[0] > 128 || v.ne[0] > 128) return false;
    if ((k.nb[1] % 16) || (k.nb[2] % 16) || (v.nb[1] % 16) || (v.nb[2] % 16) || (((uintptr_t) k.data | (uintptr_t) v.data | (uintptr_t) dst.data) & 15)) return false;
    if ((dst.nb[1] % 16) || (dst.nb[2] % 16)) return false;
    return true;
}

static bool attn_f32_type_ok(int t) { return t == GGML_TYPE_F32 || t == GGML_TYPE_BF16 || t == GGML_TYPE_F16; }

// may launch_attn_f32 serve this op?  q f32 [DK, n_q, H], k [DK, n_kv, G], v [DV, n_kv, G] of one type each, rows contiguous, one batch
bool attn_f32_applies(const tdesc & q, const tdesc & k, const tdesc & v, const tdesc * mask, const tdesc & dst) {
    if (q.type != GGML_TYPE_F32 || dst.type != GGML_TYPE_F32 || !attn_f32_type_ok(k.type) || !attn_f32_type_ok(v.type)) return false;
    if (q.ne[0] != k.ne[0] || k.ne[1] != v.ne[1] || k.ne[2] != v.ne[2] || k.ne[2] <= 0 || q.ne[2] % k.ne[2] != 0) return false;
    if (q.ne[0] < 1 || q.ne[0] > ATTN_F32_MAX_D || v.ne[0] < 1 || v.ne[0] > ATTN_F32_MAX_D) return false;
    if (q.ne[3] != 1 || k.ne[3] != 1 || v.ne[3] != 1) return false;
    if (q.nb[0] != 4 || dst.nb[0] != 4 || k.nb[0] != (k.type == GGML_TYPE_F32 ? 4 : 2) || v.nb[0] != (v.type == GGML_TYPE_F32 ? 4 : 2)) return false;
    if (dst.ne[0] != v.ne[0] || dst.ne[1] != q.ne[2] || dst.ne[2] != q.ne[1]) return false;
    if (mask && ((mask->type != GGML_TYPE_F16 && mask->type != GGML_TYPE_F32) || mask->ne[0] < k.ne[1] || mask->ne[1] < q.ne[1] || mask->ne[2] != 1 || mask->ne[3] != 1)) return false;
    return true;
}

template <int KT, int VT>
static void attn_f32_launch_t(hipStream_t s, const tdesc & q, const tdesc & k, const tdesc & v, const tdesc * mask, const float * sinks, const float * r12, const tdesc & dst, float scale,
                              const float * sig, float softcap) {
    const int64_t n_q = q.ne[1], H = q.ne[2];
    const int DK = (int) q.ne[0], DV = (int) v.ne[0];
    if constexpr (KT == GGML_TYPE_BF16 && VT == GGML_TYPE_BF16) {
        static const bool mma_on = !getenv("GGML_MI355X_ATTN_MMA") || atoi(getenv("GGML_MI355X_ATTN_MMA")) != 0;
        if (mma_on && attn_mma_bf16_wide_ok(q, k, v, mask, dst)) {  // one shared key/value head with wide rows (latent attention): four waves per 32 (token, head) pairs
            const dim3 grid((unsigned) ((n_q * H + 31) / 32));
            const int dkq = ((DK + 15) / 16 + 3) / 4, dvq = ((DV + 31) / 32 + 3) / 4;  // per wave: 16-entry key groups (<= 10), 32-entry value tiles (<= 4)
#define MI_ATT_WIDE(A, B) hipLaunchKernelGGL((k_attn_mma_bf16_wide<A, B>), grid, dim3(256), 0, s, q, k, v, *mask, sinks, r12, dst, scale, sig, softcap)
            const int a = dkq <= 3 ? 3 : (dkq <= 5 ? 5 : 10), b = dvq <= 1 ? 1 : (dvq <= 2 ? 2 : 4);
            if (a == 3 && b == 1) MI_ATT_WIDE(3, 1); else if (a == 3 && b == 2) MI_ATT_WIDE(3, 2); else if (a == 3) MI_ATT_WIDE(3, 4);
            else if (a == 5 && b == 1) MI_ATT_WIDE(5, 1); else if (a == 5 && b == 2) MI_ATT_WIDE(5, 2); else if (a == 5) MI_ATT_WIDE(5, 4);
            else if (b == 1) MI_ATT_WIDE(10, 1); else if (b == 2) MI_ATT_WIDE(10, 2); else MI_ATT_WIDE(10, 4);
#undef MI_ATT_WIDE
            return;
        }
        if (mma_on && attn_mma_bf16_ok(q, k, v, mask, dst)) {  // prompt portions over a bf16 cache: the matrix cores
            // waves per workgroup: four share a staged V^T block; two when four would leave most of the chip's 256 CUs without a workgroup (measured at 512 queries x 16
            // heads: 1.87 ms for 16 launches with two waves, 2.12 with four, 1.99 with one)
            int nw = ((n_q + 127) / 128) * H < 256 ? 2 : 4;
            static const int nw_env = getenv("GGML_MI355X_ATTN_NW") ? atoi(getenv("GGML_MI355X_ATTN_NW")) : 0;
            if (nw_env == 1 || nw_env == 2 || nw_env == 4) nw = nw_env;
            while (nw > 1 && 32 * (nw / 2) >= n_q) nw >>= 1;  // (no more waves than the batch has groups of 32 queries)
            const dim3 grid((unsigned) ((n_q + 32 * nw - 1) / (32 * nw)), (unsigned) H);
            const dim3 block((unsigned) (64 * nw));
            const int dk16 = (DK + 15) / 16, dvt = (DV + 31) / 32;
#define MI_ATT_MMA(A, B) hipLaunchKernelGGL((k_attn_mma_bf16<A, B>), grid, block, 0, s, q, k, v, *mask, sinks, r12, dst, scale, sig, softcap)
            const int a = dk16 <= 2 ? 2 : (dk16 <= 4 ? 4 : 8), b = dvt <= 1 ? 1 : (dvt <= 2 ? 2 : 4);
            if (a == 2 && b == 1) MI_ATT_MMA(2, 1); else if (a == 2 && b == 2) MI_ATT_MMA(2, 2); else if (a == 2) MI_ATT_MMA(2, 4);
            else if (a == 4 && b == 1) MI_ATT_MMA(4, 1); else if (a == 4 && b == 2) MI_ATT_MMA(4, 2); else if (a == 4) MI_ATT_MMA(4, 4);
            else if (b == 1) MI_ATT_MMA(8, 1); else if (b == 2) MI_ATT_MMA(8, 2); else MI_ATT_MMA(8, 4);
#undef MI_ATT_MMA
            return;
        }
    }
    // the tile kernel: batches of 32 queries and more under a mask, head sizes up to 128 (its LDS: 64 cells of K and V plus 64 queries as f32)
    if (mask && n_q >= 32 && DK <= 128 && DV <= 128) {
        const dim3 grid((unsigned) ((n_q + 63) / 64), (unsigned) H);
        auto go = [&](auto kern, int dkp, int dvp) {
            const size_t lds = ((size_t) 64 * (dkp + 1) + (size_t) 64 * dvp + (size_t) 64 * dkp) * sizeof(float);
            // (more than the 64 KB a kernel gets by default: up to 97 KB of the CU's 160 KB; the attribute is per device and cheap to set again)
            if (lds > 48 * 1024) (void) hipFuncSetAttribute((const void *) kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds);
            hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, q, k, v, *mask, sinks, r12, dst, scale, sig, softcap);
        };
        const bool k64 = DK <= 64, v64 = DV <= 64;
        if (k64 && v64) go(k_attn_f32_tile<KT, VT, 64, 64>, 64, 64);
        else if (k64) go(k_attn_f32_tile<KT, VT, 64, 128>, 64, 128);
        else if (v64) go(k_attn_f32_tile<KT, VT, 128, 64>, 128, 64);
        else go(k_attn_f32_tile<KT, VT, 128, 128>, 128, 128);
        return;
    }
    hipLaunchKernelGGL((k_attn_f32_rows<KT, VT>), dim3((unsigned) n_q, (unsigned) H), dim3(256), 0, s, q, k, v, mask ? *mask : q, mask ? 1 : 0, sinks, r12, dst, scale, sig, softcap);
}

void launch_attn_f32(hipStream_t s, const tdesc & q, const tdesc & k, const tdesc & v, const tdesc * mask, const float * sinks, const float * r12, const tdesc & dst, float scale,
                     const float * sig, float softcap) {
    if (q.ne[1] == 0 || q.ne[2] == 0) return;
#define MI_ATTN_F32_CASE(KT, VT) if (k.type == KT && v.type == VT) { attn_f32_launch_t<KT, VT>(s, q, k, v, mask, sinks, r12, dst, scale, sig, softcap); return; }
    MI_ATTN_F32_CASE(GGML_TYPE_F32, GGML_TYPE_F32)
    MI_ATTN_F32_CASE(GGML_TYPE_BF16, GGML_TYPE_BF16)
    MI_ATTN_F32_CASE(GGML_TYPE_F16, GGML_TYPE_F16)
    MI_ATTN_F32_CASE(GGML_TYPE_F32, GGML_TYPE_BF16)
    MI_ATTN_F32_CASE(GGML_TYPE_BF16, GGML_TYPE_F32)
    MI_ATTN_F32_CASE(GGML_TYPE_F32, GGML_TYPE_F16)
    MI_ATTN_F32_CASE(GGML_TYPE_F16, GGML_TYPE_F32)
    MI_ATTN_F32_CASE(GGML_TYPE_BF16, GGML_TYPE_F16)
    MI_ATTN_F32_CASE(GGML_TYPE_F16, GGML_TYPE_BF16)
#undef MI_ATTN_F32_CASE
}

MI_TU_TOUCH(attn_f32)

}  // namespace mi355x
