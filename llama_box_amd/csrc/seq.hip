// seq.hip — layers that carry STATE from token to token of a sequence, over a batch that mixes sequences freely (prompt portions of some beside
// single tokens of others).  The scheduler describes the batch with four small integer inputs:
//   hist [hs, T]      for token t and d = 1 .. hs: where the d-th token BEFORE t of the same sequence is found — a row of this batch (>= 0), nowhere (-1: before
//                     the sequence's start, reads as zero), or the sequence's state (-2 - (slot * 64 + age): the age-th most recent token before this batch);
//   upd  [hs, n_seq]  the same codes for the state AFTER the batch: entry a of sequence s is where its new age-a token comes from;
//   tok  [T]          the batch rows grouped by sequence, each group in position order;
//   info [4, n_seq]   per sequence of the batch: (first entry of its group in tok, number of entries, state slot, 1 when the sequence starts in this batch).
// A sequence that starts reads no state at all (zeros), so a slot taken over by a new request needs no clearing.
//
// Kernels:
//   k_seq_conv        short causal convolution per channel over a sequence's history (taps inputs, the last one the token's own), optionally followed by SiLU;
//                     several weight sets over the same input give several outputs (a token shift h + (h_prev - h) mu is the 2-tap case with weights (mu, 1 - mu))
//   k_seq_conv_store  the last taps - 1 inputs of every sequence of the batch become its state
//   k_seq_recurrence<SEQ_WKV6>   o_t = (S + diag(u) k v^T)^T r;  S <- diag(w) S + k v^T, w = exp(-exp(w_pre + w0)) per key channel
//   k_seq_recurrence<SEQ_DELTA>  gated delta rule: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q — unit-length q, k, sigmoid beta and the decay
//                     g = exp(-exp(A_log) softplus(a + dt_bias)) computed here from the raw projections
//   k_seq_recurrence<SEQ_DELTA_CH>  the delta rule with ONE DECAY PER KEY CHANNEL: S <- diag(g) S with g = exp(-exp(A_log) softplus(a + dt_bias)) per (head, key row), the
//                     raw a [DK H, T] being a projection of its own; beta = sigmoid(b_pre) from a [H, T] projection; the rest as SEQ_DELTA
//   k_seq_recurrence<SEQ_SSD>    state-space duality (Mamba-2): dt = softplus(dt_pre + dt_bias); S <- exp(-exp(A_log) dt) S + dt B x^T; y = S^T C + D x, with B as the keys,
//                     C as the queries (grouped: head h reads group h / (H / G)) and x as the values
//   k_seq_recurrence<SEQ_MLSTM>  matrix memory with exponential gates under a running maximum m: m' = max(f + m, i); S <- e^(f + m - m') S + e^(i - m') k v^T; n likewise with k;
//                     o = S^T q / (max(|n . q|, e^(-m')) + 1e-6); log gates capped by cap tanh(. / cap), f through log-sigmoid
// All arithmetic is f32; the state is f32.  The three recurrences share one thread layout: a wave per (sequence of the batch, head, 4 value columns); value column j
// of the head's state matrix is held by SIXTEEN neighbouring lanes (a DPP row), each owning a sixteenth of the key rows (neighbours) in registers; dot products over the key
// rows are partial sums per lane joined across the sixteen by four DPP permutations (every lane then holds the same sum).  The vectors of several tokens are staged in
// LDS a block ahead.  In memory a head's matrix is kept in the order the lanes read it ([register][column][ks]: one coalesced load per register).
#include <algorithm>
#include <cstdlib>

#include "dev_util.h"
#include "kernels.h"

namespace mi355x {

constexpr int SEQ_MAX_TAPS = 16;
constexpr int SEQ_MAX_DK = 256;  // key rows of a head (16 lanes x up to 16 rows each)

__device__ __forceinline__ float seq_hist_value(const int code, const int c, const int64_t C, const int taps, const char * __restrict__ xdata, const int64_t x_nb1,
                                                const float * __restrict__ state) {
    if (code >= 0) return ((const float *) (xdata + (int64_t) code * x_nb1))[c];
    if (code == -1) return 0.0f;
    const int cd = -2 - code, slot = cd >> 6, age = cd & 63;
    return state[((int64_t) slot * (taps - 1) + age) * C + c];
}

__device__ __forceinline__ float seq_silu(const float z) { return z / (1.0f + expf(-z)); }

// y[c, t, m] = act(sum_j w[j, c, m] * x_(t - (taps - 1 - j))[c] + bias[c, m])   (bias may be null)
__global__ void __launch_bounds__(256) k_seq_conv(const tdesc x, const float * __restrict__ w, const float * __restrict__ bias, const float * __restrict__ state,
                                                  const int32_t * __restrict__ hist, const int hs, const tdesc dst, const int taps, const int act) {
    const int64_t C = x.ne[0], t = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    float xv[SEQ_MAX_TAPS];  // xv[d]: the input d tokens back
    xv[0] = ((const float *) (x.data + t * x.nb[1]))[c];
#pragma unroll
    for (int d = 1; d < SEQ_MAX_TAPS; ++d) xv[d] = d < taps ? seq_hist_value(hist[t * hs + d - 1], c, C, taps, x.data, x.nb[1], state) : 0.0f;
    for (int64_t m = 0; m < dst.ne[2]; ++m) {
        const float * __restrict__ wc = w + (m * C + c) * taps;
        float y = 0.0f;
#pragma unroll
        for (int d = SEQ_MAX_TAPS - 1; d >= 0; --d)
            if (d < taps) y = fmaf(wc[taps - 1 - d], xv[d], y);  // oldest input first
        if (bias) y += bias[m * C + c];
        ((float *) (dst.data + t * dst.nb[1] + m * dst.nb[2]))[c] = act ? seq_silu(y) : y;
    }
}

__global__ void __launch_bounds__(256) k_seq_conv_store(const tdesc x, float * __restrict__ state, const int32_t * __restrict__ upd, const int hs, const int32_t * __restrict__ info,
                                                        const int taps) {
    const int64_t C = x.ne[0], s = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int slot = info[4 * s + 2];
    float nv[SEQ_MAX_TAPS - 1];
#pragma unroll
    for (int a = 0; a < SEQ_MAX_TAPS - 1; ++a) nv[a] = a < taps - 1 ? seq_hist_value(upd[s * hs + a], c, C, taps, x.data, x.nb[1], state) : 0.0f;
#pragma unroll
    for (int a = 0; a < SEQ_MAX_TAPS - 1; ++a)
        if (a < taps - 1) state[((int64_t) slot * (taps - 1) + a) * C + c] = nv[a];  // (every value was read before the first is written: the rows shift in place)
}

void launch_seq_conv(hipStream_t s, const tdesc & x, const float * w, const float * bias, const float * state, const int32_t * hist, int hs, const tdesc & dst, int taps, int act) {
    if (x.ne[1] == 0 || x.ne[0] == 0) return;
    hipLaunchKernelGGL(k_seq_conv, dim3((unsigned) ((x.ne[0] + 255) / 256), (unsigned) x.ne[1]), dim3(256), 0, s, x, w, bias, state, hist, hs, dst, taps, act);
}
void launch_seq_conv_store(hipStream_t s, const tdesc & x, float * state, const int32_t * upd, int hs, const int32_t * info, int n_seqs, int taps) {
    if (n_seqs == 0 || x.ne[0] == 0 || taps < 2) return;
    hipLaunchKernelGGL(k_seq_conv_store, dim3((unsigned) ((x.ne[0] + 255) / 256), (unsigned) n_seqs), dim3(256), 0, s, x, state, upd, hs, info, taps);
}

// ------------------------------------------------------------------------------------------------ the recurrences
__device__ __forceinline__ float quad_sum(float x) {  // sum over the 16 lanes of a row (the lanes of one value column); every lane gets the same bits
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0xB1, 0xF, 0xF, true));   // quad lanes (1, 0, 3, 2)
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x4E, 0xF, 0xF, true));   // quad lanes (2, 3, 0, 1): the four hold their quad's sum
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x141, 0xF, 0xF, true));  // mirrored within each half row: the other quad of the half
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x140, 0xF, 0xF, true));  // mirrored within the row: the other half
    return x;
}
__device__ __forceinline__ float seq_softplus(const float z) { return fmaxf(z, 0.0f) + log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float seq_log_sigmoid(const float z) { return fminf(z, 0.0f) - log1pf(expf(-fabsf(z))); }


// One WAVE per (sequence of the batch, head, group of 4 value columns).  The tokens' vectors come in blocks of TB tokens: while block b is worked on out of LDS, block
// b + 1 travels from memory into registers (one trip to memory per block, not per token) and is written to the other LDS buffer at the end; the batch rows of block b + 2
// are fetched at the same time, so that no load ever waits for an address that is itself on its way.  A token's entries in a block: k [DK], q [DK], (wkv6: decay [DK]),
// the wave's 4 values, (delta / state space / matrix memory: the head's raw gates).
constexpr int SEQ_COLS = 4;        // value columns of a wave
constexpr int SEQ_LPC = 16;        // lanes per value column: each owns a sixteenth of the key rows
constexpr int SEQ_NV = 32;         // registers a lane lends to the block on its way
constexpr int SEQ_MAX_TB = 16;     // tokens of a block at most
constexpr int SEQ_DECAY_PREPASS_MIN = 32;  // batches of this many tokens and more compute the channel decays in a pass of their own

// key rows a lane owns: a sixteenth of the head's rows, rounded up to whole groups of four (its rows are neighbours, read from LDS sixteen bytes at a time)
static inline __host__ __device__ int seq_rows_per_lane(const int DK) { return (((DK + SEQ_LPC - 1) / SEQ_LPC) + 3) / 4 * 4; }
// which kinds carry a decay per key channel among a token's entries, and which carry raw gates of the head
static inline __host__ __device__ bool seq_has_w(const int kind) { return kind == SEQ_WKV6 || kind == SEQ_DELTA_CH; }
static inline __host__ __device__ bool seq_has_gates(const int kind) { return kind != SEQ_WKV6; }
// floats a token occupies in a staged block (at least a wave's stride: the walk over a block's entries then crosses at most one token per step)
static inline __host__ __device__ int seq_per_tok(const int kind, const int DK) {
    const int n = (seq_has_w(kind) ? 3 : 2) * SEQ_LPC * seq_rows_per_lane(DK) + SEQ_COLS + (seq_has_gates(kind) ? 4 : 0);
    return n > 64 ? n : 64;
}

template <int KIND, int R, bool EXACT>   // R: key rows per lane at most (a multiple of 4); EXACT: exactly R (no test around a group of four rows)
__global__ void __launch_bounds__(64) k_seq_recurrence(const seq_rec_args A, const int TB) {
    __shared__ __attribute__((aligned(16))) float blk[2][SEQ_NV * 64];
    __shared__ int rows_of[2][SEQ_MAX_TB];
    const int s = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * SEQ_COLS, lane = threadIdx.x;
    const int begin = A.info[4 * s], count = A.info[4 * s + 1], slot = A.info[4 * s + 2], reset = A.info[4 * s + 3];
    const int DK = A.DK, DV = A.DV, H = A.H;
    const int j = j0 + (lane >> 4), ks = lane & (SEQ_LPC - 1);
    const bool col = j < DV;
    const int RL = seq_rows_per_lane(DK), KP = SEQ_LPC * RL;  // lane ks owns rows ks RL .. ks RL + RL - 1; a token's key-sized vectors are padded with zeros to KP entries
    const int kh = KIND == SEQ_WKV6 ? h : h / (H / A.G);
    constexpr bool HAS_W = KIND == SEQ_WKV6 || KIND == SEQ_DELTA_CH, HAS_G = KIND != SEQ_WKV6, IS_DELTA = KIND == SEQ_DELTA || KIND == SEQ_DELTA_CH;
    const int off_w = 2 * KP, off_v = HAS_W ? 3 * KP : 2 * KP, off_g = off_v + SEQ_COLS;
    const int per_tok = seq_per_tok(KIND, DK);
    float * __restrict__ Sm = A.state + (int64_t) slot * A.state_stride + (int64_t) h * RL * DV * SEQ_LPC;
    float * __restrict__ Nm = A.state + (int64_t) slot * A.state_stride + (int64_t) H * RL * DV * SEQ_LPC + (int64_t) h * DK;
    float * __restrict__ Mm = A.state + (int64_t) slot * A.state_stride + (int64_t) H * RL * DV * SEQ_LPC + (int64_t) H * DK + h;
    float S[R], nn[R], uu[R];
#pragma unroll
    for (int ii = 0; ii < R; ++ii) {
        // (no branch around a load: an entry that does not exist reads entry 0 and is dropped — the loads of all registers are then in flight together)
        const int i = ks * RL + ii;
        const bool ok = ii < RL && i < DK;
        const float sv = Sm[(ok && col) ? ((int64_t) ii * DV + j) * SEQ_LPC + ks : 0];
        S[ii] = (ok && col && !reset) ? sv : 0.0f;
        if (KIND == SEQ_MLSTM) { const float nv = Nm[ok ? i : 0]; nn[ii] = (ok && !reset) ? nv : 0.0f; } else nn[ii] = 0.0f;
        if (KIND == SEQ_WKV6) { const float uv = A.p1[h * DK + (ok ? i : 0)]; uu[ii] = ok ? uv : 0.0f; } else uu[ii] = 0.0f;
    }
    float mrun = (KIND == SEQ_MLSTM && !reset) ? *Mm : 0.0f;
    const float a_exp = (IS_DELTA || KIND == SEQ_SSD) ? expf(A.p0[h]) : 0.0f;
    const float dt_b = (KIND == SEQ_DELTA || KIND == SEQ_SSD) ? A.p0[H + h] : 0.0f;
    const float d_skip = KIND == SEQ_SSD ? A.p0[2 * H + h] : 0.0f;
    const float bi = KIND == SEQ_MLSTM ? A.p0[h] : 0.0f, bf = KIND == SEQ_MLSTM ? A.p0[H + h] : 0.0f;

    // entry e = lane + 64 i of a block (token u = e / per_tok, field f = e % per_tok) read from memory; `rows`: the block's batch rows
    auto fetch = [&](const int * rows, const int n_tok, float (&pre)[SEQ_NV]) {
        int u = lane >= per_tok ? 1 : 0, f = lane >= per_tok ? lane - per_tok : lane;  // (no loop inside: the 32 steps are one run of straight code)
#pragma unroll
        for (int i = 0; i < SEQ_NV; ++i) {
            // which tensor, which entry: selected without branches, an entry that does not exist reads entry 0 of the block's first token (32 loads in flight together)
            const bool is_k = f < KP, is_q = !is_k && f < 2 * KP, is_w = HAS_W && !is_k && !is_q && f < off_v, is_v = !is_k && !is_q && !is_w && f < off_g;
            const int fe = is_k ? f : is_q ? f - KP : is_w ? f - off_w : is_v ? f - off_v : f - off_g;
            // gates of the head: two raw projections (delta: b, a; matrix memory: i, f), one of its own tensor (channel decay: b), or one read twice (state space: dt)
            const bool valid = u < n_tok && (is_v ? j0 + fe < DV : (is_k || is_q || is_w) ? fe < DK : (HAS_G && fe < (KIND == SEQ_DELTA_CH ? 1 : 2)));
            const bool is_gate = !is_k && !is_q && !is_w && !is_v;
            const char * base = is_k ? A.k.data : is_q ? A.q.data : is_v ? A.v.data : (KIND == SEQ_DELTA_CH && is_gate) ? A.b.data : A.g.data;
            const int64_t nb1 = is_k ? A.k.nb[1] : is_q ? A.q.nb[1] : is_v ? A.v.nb[1] : (KIND == SEQ_DELTA_CH && is_gate) ? A.b.nb[1] : A.g.nb[1];
            const int idx = (is_k || is_q) ? kh * DK + fe : is_w ? h * DK + fe : is_v ? h * DV + j0 + fe : (KIND == SEQ_DELTA_CH || KIND == SEQ_SSD) ? h : fe * H + h;
            const int64_t t = rows[valid ? u : 0];
            float val = ((const float *) (base + t * nb1))[valid ? idx : 0];
            if (HAS_W) {  // the decay's offset: w0 (time mixing), or the dt_bias entries behind the heads' A_log (channel decay)
                const float off = A.p0[(is_w && valid) ? (KIND == SEQ_DELTA_CH ? H : 0) + h * DK + fe : 0];
                val = (is_w && !(KIND == SEQ_DELTA_CH && A.w_ready)) ? val + off : val;  // (w_ready: the operand already holds the decays themselves)
            }
            pre[i] = valid ? val : 0.0f;
            f += 64;
            const bool over = f >= per_tok;
            f = over ? f - per_tok : f;
            u = over ? u + 1 : u;
        }
    };
    auto park = [&](float * dstb, const float (&pre)[SEQ_NV]) {
        int f = lane >= per_tok ? lane - per_tok : lane;
#pragma unroll
        for (int i = 0; i < SEQ_NV; ++i) {
            if (lane + 64 * i < TB * per_tok)
                dstb[lane + 64 * i] = (KIND == SEQ_WKV6 && f >= off_w && f < off_v) ? expf(-expf(pre[i])) : pre[i];
            f += 64;
            f = f >= per_tok ? f - per_tok : f;
        }
    };
    // the raw gates of a parked block become what the recurrence uses — (beta, decay) or the capped log gates — once per block, two lanes a token, instead of in
    // every token's own chain of instructions (the same formulas on the same values)
    auto finish_gates = [&](float * dstb) {
        if (HAS_G && lane < 2 * TB) {
            float * gp = dstb + (lane >> 1) * per_tok + off_g + (lane & 1);
            const float x = *gp;
            float y;
            if (KIND == SEQ_DELTA) y = (lane & 1) ? expf(-a_exp * seq_softplus(x + dt_b)) : 1.0f / (1.0f + expf(-x));
            else if (KIND == SEQ_DELTA_CH) y = (lane & 1) ? x : 1.0f / (1.0f + expf(-x));
            else if (KIND == SEQ_SSD) { const float dt = seq_softplus(x + dt_b); y = (lane & 1) ? expf(-a_exp * dt) : dt; }  // (step size, decay)
            else y = (lane & 1) ? seq_log_sigmoid(A.cap * tanhf((x + bf) / A.cap)) : A.cap * tanhf((x + bi) / A.cap);
            *gp = y;
        }
    };
    // channel decay: the parked raw values (projection + offset) of a block's n_tok tokens become exp(-e^A softplus(.)) — the lanes walk over the DK real entries of
    // every token only, so the softplus and the two exponentials are paid once per entry (not once per staged float)
    auto finish_decay = [&](float * dstb, const int n_tok) {
        if (KIND == SEQ_DELTA_CH && !A.w_ready)
            for (int idx = lane; idx < n_tok * DK; idx += 64) {
                const int u = idx / DK, fe = idx - u * DK;
                float * wp = dstb + u * per_tok + off_w + fe;
                *wp = expf(-a_exp * seq_softplus(*wp));
            }
    };
    float pre[SEQ_NV];
    if (lane < SEQ_MAX_TB) {
        rows_of[0][lane] = lane < count ? A.tok[begin + lane] : 0;
        rows_of[1][lane] = TB + lane < count ? A.tok[begin + TB + lane] : 0;
    }
    __syncthreads();
    fetch(rows_of[0], min(TB, count), pre);
    park(blk[0], pre);
    __syncthreads();
    finish_gates(blk[0]);
    finish_decay(blk[0], min(TB, count));
    __syncthreads();
    for (int b0 = 0, b = 0; b0 < count; b0 += TB, ++b) {
        const int n_here = min(TB, count - b0), n_next = min(TB, count - b0 - TB);
        const float * cur = blk[b & 1];
        const int * trow = rows_of[b & 1];
        int row_after = 0;
        if (n_next > 0) {
            fetch(rows_of[(b + 1) & 1], n_next, pre);
            if (lane < TB && b0 + 2 * TB + lane < count) row_after = A.tok[begin + b0 + 2 * TB + lane];
        }
        if (KIND == SEQ_SSD) {
            // the state's update waits for nothing but the state (the read-out is beside the chain), so what a token costs is the trip to LDS for its vectors: the next
            // token's are requested before the current token's arithmetic (the delta rules and the matrix memory, whose tokens are chains of dependent reductions, gain
            // nothing from the same: measured, and left as they are)
            float4 nk[R / 4], nq[R / 4];
            float nv, ng0, ng1;
            auto stage = [&](const int u) {
                const float * lt = cur + u * per_tok;
                const float4 * k4 = (const float4 *) (lt + ks * RL), * q4 = (const float4 *) (lt + KP + ks * RL);
#pragma unroll
                for (int m = 0; m < R / 4; ++m) {
                    nk[m] = make_float4(0.f, 0.f, 0.f, 0.f);
                    nq[m] = nk[m];
                    if (EXACT || 4 * m < RL) { nk[m] = k4[m]; nq[m] = q4[m]; }
                }
                nv = lt[off_v + (lane >> 4)];
                ng0 = lt[off_g];
                ng1 = lt[off_g + 1];
            };
            stage(0);
            for (int u = 0; u < n_here; ++u) {
                float4 kk[R / 4], cq[R / 4];
#pragma unroll
                for (int m = 0; m < R / 4; ++m) { kk[m] = nk[m]; cq[m] = nq[m]; }
                const float vj = nv, dtv = ng0 * vj, dec = ng1;
                if (u + 1 < n_here) stage(u + 1);
                float p0 = 0.0f, p1 = 0.0f, p2 = 0.0f, p3 = 0.0f;
#pragma unroll
                for (int m = 0; m < R / 4; ++m) {
                    if (EXACT || 4 * m < RL) {
                        S[4 * m] = fmaf(kk[m].x, dtv, dec * S[4 * m]);
                        S[4 * m + 1] = fmaf(kk[m].y, dtv, dec * S[4 * m + 1]);
                        S[4 * m + 2] = fmaf(kk[m].z, dtv, dec * S[4 * m + 2]);
                        S[4 * m + 3] = fmaf(kk[m].w, dtv, dec * S[4 * m + 3]);
                        p0 = fmaf(S[4 * m], cq[m].x, p0);
                        p1 = fmaf(S[4 * m + 1], cq[m].y, p1);
                        p2 = fmaf(S[4 * m + 2], cq[m].z, p2);
                        p3 = fmaf(S[4 * m + 3], cq[m].w, p3);
                    }
                }
                const float o = fmaf(d_skip, vj, quad_sum((p0 + p1) + (p2 + p3)));
                if (col && ks == 0) ((float *) (A.dst.data + (int64_t) h * A.dst.nb[1] + (int64_t) trow[u] * A.dst.nb[2]))[j] = o;
            }
        } else
        for (int u = 0; u < n_here; ++u) {
            const float * lt = cur + u * per_tok;
            const float4 * k4 = (const float4 *) (lt + ks * RL), * q4 = (const float4 *) (lt + KP + ks * RL), * w4 = (const float4 *) (lt + off_w + ks * RL);
            const float vj = lt[off_v + (lane >> 4)];
            float o = 0.0f;
            if (KIND == SEQ_WKV6) {
                float p0 = 0.0f, p1 = 0.0f, p2 = 0.0f, p3 = 0.0f;
#pragma unroll
                for (int m = 0; m < R / 4; ++m) {
                    if (EXACT || 4 * m < RL) {
                        const float4 kk = k4[m], rq = q4[m], ww = w4[m];
                        const float kv0 = kk.x * vj, kv1 = kk.y * vj, kv2 = kk.z * vj, kv3 = kk.w * vj;
                        p0 = fmaf(fmaf(uu[4 * m], kv0, S[4 * m]), rq.x, p0);
                        p1 = fmaf(fmaf(uu[4 * m + 1], kv1, S[4 * m + 1]), rq.y, p1);
                        p2 = fmaf(fmaf(uu[4 * m + 2], kv2, S[4 * m + 2]), rq.z, p2);
                        p3 = fmaf(fmaf(uu[4 * m + 3], kv3, S[4 * m + 3]), rq.w, p3);
                        S[4 * m] = fmaf(ww.x, S[4 * m], kv0);
                        S[4 * m + 1] = fmaf(ww.y, S[4 * m + 1], kv1);
                        S[4 * m + 2] = fmaf(ww.z, S[4 * m + 2], kv2);
                        S[4 * m + 3] = fmaf(ww.w, S[4 * m + 3], kv3);
                    }
                }
                o = quad_sum((p0 + p1) + (p2 + p3));
            } else if (IS_DELTA) {
                const float beta = lt[off_g], gdec = lt[off_g + 1];
                float kn[R], qn[R];
                float k2a = 0.0f, k2b = 0.0f, q2a = 0.0f, q2b = 0.0f;
#pragma unroll
                for (int m = 0; m < R / 4; ++m) {
                    float4 kk = make_float4(0.f, 0.f, 0.f, 0.f), qq = kk;
                    if (EXACT || 4 * m < RL) { kk = k4[m]; qq = q4[m]; }
                    if (KIND == SEQ_DELTA_CH && (EXACT || 4 * m < RL)) {  // one decay per key row: applied here, ahead of the unit lengths (it waits for nothing but its own load)
                        const float4 ww = w4[m];
                        S[4 * m] *= ww.x; S[4 * m + 1] *= ww.y; S[4 * m + 2] *= ww.z; S[4 * m + 3] *= ww.w;
                    }
                    kn[4 * m] = kk.x; kn[4 * m + 1] = kk.y; kn[4 * m + 2] = kk.z; kn[4 * m + 3] = kk.w;
                    qn[4 * m] = qq.x; qn[4 * m + 1] = qq.y; qn[4 * m + 2] = qq.z; qn[4 * m + 3] = qq.w;
                    k2a = fmaf(kk.x, kk.x, fmaf(kk.z, kk.z, k2a));
                    k2b = fmaf(kk.y, kk.y, fmaf(kk.w, kk.w, k2b));
                    q2a = fmaf(qq.x, qq.x, fmaf(qq.z, qq.z, q2a));
                    q2b = fmaf(qq.y, qq.y, fmaf(qq.w, qq.w, q2b));
                }
                const float kinv = 1.0f / sqrtf(quad_sum(k2a + k2b) + 1e-6f), qinv = 1.0f / sqrtf(quad_sum(q2a + q2b) + 1e-6f) * A.qscale;
                float d0 = 0.0f, d1 = 0.0f, d2 = 0.0f, d3 = 0.0f;
#pragma unroll
                for (int m = 0; m < R / 4; ++m) {
                    if (EXACT || 4 * m < RL) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) { kn[4 * m + e] *= kinv; if (KIND == SEQ_DELTA) S[4 * m + e] *= gdec; }
                        d0 = fmaf(S[4 * m], kn[4 * m], d0);
                        d1 = fmaf(S[4 * m + 1], kn[4 * m + 1], d1);
                        d2 = fmaf(S[4 * m + 2], kn[4 * m + 2], d2);
                        d3 = fmaf(S[4 * m + 3], kn[4 * m + 3], d3);
                    }
                }
                const float uw = beta * (vj - quad_sum((d0 + d1) + (d2 + d3)));
                float p0 = 0.0f, p1 = 0.0f, p2 = 0.0f, p3 = 0.0f;
#pragma unroll
                for (int m = 0; m < R / 4; ++m) {
                    if (EXACT || 4 * m < RL) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) S[4 * m + e] = fmaf(kn[4 * m + e], uw, S[4 * m + e]);
                        p0 = fmaf(S[4 * m], qn[4 * m] * qinv, p0);
                        p1 = fmaf(S[4 * m + 1], qn[4 * m + 1] * qinv, p1);
                        p2 = fmaf(S[4 * m + 2], qn[4 * m + 2] * qinv, p2);
                        p3 = fmaf(S[4 * m + 3], qn[4 * m + 3] * qinv, p3);
                    }
                }
                o = quad_sum((p0 + p1) + (p2 + p3));
            } else {
                const float ig = lt[off_g], fg = lt[off_g + 1];
                const float m_new = fmaxf(fg + mrun, ig);
                const float ea = expf(fg + mrun - m_new), eb = expf(ig - m_new);
                mrun = m_new;
                float n0 = 0.0f, n1 = 0.0f, e0 = 0.0f, e1 = 0.0f;
#pragma unroll
                for (int m = 0; m < R / 4; ++m) {
                    if (EXACT || 4 * m < RL) {
                        const float4 kk = k4[m], qq = q4[m];
                        const float kf[4] = {kk.x, kk.y, kk.z, kk.w}, qf[4] = {qq.x * A.qscale, qq.y * A.qscale, qq.z * A.qscale, qq.w * A.qscale};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            S[4 * m + e] = fmaf(eb * kf[e], vj, ea * S[4 * m + e]);
                            nn[4 * m + e] = fmaf(eb, kf[e], ea * nn[4 * m + e]);
                        }
                        n0 = fmaf(S[4 * m], qf[0], fmaf(S[4 * m + 2], qf[2], n0));
                        n1 = fmaf(S[4 * m + 1], qf[1], fmaf(S[4 * m + 3], qf[3], n1));
                        e0 = fmaf(nn[4 * m], qf[0], fmaf(nn[4 * m + 2], qf[2], e0));
                        e1 = fmaf(nn[4 * m + 1], qf[1], fmaf(nn[4 * m + 3], qf[3], e1));
                    }
                }
                const float num = quad_sum(n0 + n1), den = quad_sum(e0 + e1);
                o = num / (fmaxf(fabsf(den), expf(-m_new)) + 1e-6f);
            }
            if (col && ks == 0) ((float *) (A.dst.data + (int64_t) h * A.dst.nb[1] + (int64_t) trow[u] * A.dst.nb[2]))[j] = o;
        }
        __syncthreads();  // (every lane has finished with this block's batch rows before they are replaced)
        if (n_next > 0) {
            park(blk[(b + 1) & 1], pre);
            if (lane < TB) rows_of[b & 1][lane] = row_after;
            __syncthreads();
            finish_gates(blk[(b + 1) & 1]);
            finish_decay(blk[(b + 1) & 1], n_next);
        }
        __syncthreads();
    }
#pragma unroll
    for (int ii = 0; ii < R; ++ii) {
        const int i = ks * RL + ii;
        const bool ok = ii < RL && i < DK;
        if (col && ok) Sm[((int64_t) ii * DV + j) * SEQ_LPC + ks] = S[ii];
        if (KIND == SEQ_MLSTM && j0 == 0 && lane < SEQ_LPC && ok) Nm[i] = nn[ii];
    }
    if (KIND == SEQ_MLSTM && j0 == 0 && lane == 0) *Mm = mrun;
}

// the decays of the channel-decay delta rule for a whole batch at once, out[t][c] = exp(-exp(A_log[c / DK]) softplus(a[t][c] + dt_bias[c])) — the formula of the recurrence
// kernel on the same values, taken out of its token-after-token loop for prompt portions (every entry is independent of every other)
__global__ void __launch_bounds__(256) k_seq_channel_decay(const tdesc a, const float * __restrict__ p0, const int H, const int DK, float * __restrict__ out) {
    const int64_t C = (int64_t) H * DK, t = blockIdx.y;
    const int64_t c = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const float a_exp = expf(p0[c / DK]);
    const float val = ((const float *) (a.data + t * a.nb[1]))[c] + p0[H + c];
    out[t * C + c] = expf(-a_exp * seq_softplus(val));
}
size_t seq_recurrence_scratch_bytes(int kind, int H, int DK, int64_t T) { return (kind == SEQ_DELTA_CH && T >= SEQ_DECAY_PREPASS_MIN) ? (size_t) T * H * DK * sizeof(float) : 0; }

// floats of state one slot needs
int64_t seq_recurrence_state_floats(int kind, int H, int DK, int DV) {
    return (int64_t) H * seq_rows_per_lane(DK) * DV * SEQ_LPC + (kind == SEQ_MLSTM ? (int64_t) H * DK + H : 0);
}
// (a lane holds up to 64 key rows of its column; a token's entries must fit the registers a wave lends to a block)
bool seq_recurrence_ok(int DK, int DV) { return DK >= 1 && DK <= SEQ_MAX_DK && DV >= 1 && 3 * SEQ_LPC * seq_rows_per_lane(DK) + SEQ_COLS + 4 <= SEQ_NV * 64; }

template <int KIND>
static void seq_recurrence_launch(hipStream_t s, const seq_rec_args & a, int n_seqs) {
    const int RL = seq_rows_per_lane(a.DK);
    const int per_tok = seq_per_tok(KIND, a.DK);
    int TB = std::max(1, std::min(SEQ_MAX_TB, SEQ_NV * 64 / per_tok));
    static const int tb_env = getenv("GGML_MI355X_SEQ_TB") ? atoi(getenv("GGML_MI355X_SEQ_TB")) : 0;  // (lab switch: fewer tokens per block)
    if (tb_env > 0) TB = std::min(TB, tb_env);
    const dim3 grid((unsigned) n_seqs, (unsigned) a.H, (unsigned) ((a.DV + SEQ_COLS - 1) / SEQ_COLS));
#define MI_SEQ_REC(RR) do { if (RL == RR) hipLaunchKernelGGL((k_seq_recurrence<KIND, RR, true>), grid, dim3(64), 0, s, a, TB); \
                            else hipLaunchKernelGGL((k_seq_recurrence<KIND, RR, false>), grid, dim3(64), 0, s, a, TB); } while (0)
    if (RL <= 4) MI_SEQ_REC(4);
    else if (RL <= 8) MI_SEQ_REC(8);
    else MI_SEQ_REC(16);
#undef MI_SEQ_REC
}
void launch_seq_recurrence(hipStream_t s, int kind, const seq_rec_args & a_in, int n_seqs, void * scratch, size_t scratch_bytes) {
    if (n_seqs == 0 || a_in.H == 0) return;
    seq_rec_args a = a_in;
    a.w_ready = 0;
    const int64_t T = a.g.ne[1];
    const size_t need = seq_recurrence_scratch_bytes(kind, a.H, a.DK, T);
    if (need > 0 && scratch && need <= scratch_bytes) {  // a prompt portion: the decays of all its tokens in one parallel pass
        const int64_t C = (int64_t) a.H * a.DK;
        hipLaunchKernelGGL(k_seq_channel_decay, dim3((unsigned) ((C + 255) / 256), (unsigned) T), dim3(256), 0, s, a.g, a.p0, a.H, a.DK, (float *) scratch);
        a.g.data = (char *) scratch;
        a.g.nb[0] = 4;
        a.g.nb[1] = C * 4;
        a.w_ready = 1;
    }
    if (kind == SEQ_WKV6) seq_recurrence_launch<SEQ_WKV6>(s, a, n_seqs);
    else if (kind == SEQ_DELTA) seq_recurrence_launch<SEQ_DELTA>(s, a, n_seqs);
    else if (kind == SEQ_DELTA_CH) seq_recurrence_launch<SEQ_DELTA_CH>(s, a, n_seqs);
    else if (kind == SEQ_SSD) seq_recurrence_launch<SEQ_SSD>(s, a, n_seqs);
    else seq_recurrence_launch<SEQ_MLSTM>(s, a, n_seqs);
}

MI_TU_TOUCH(seq)

}  // namespace mi355x
