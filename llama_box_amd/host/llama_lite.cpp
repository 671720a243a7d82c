// llama_lite.cpp — see llama_lite.h.  Own driver: model container (synthetic or GGUF), unified KV cache,
// per-micro-batch graph construction in the op order llm_build_llama / llm_build_qwen2 emit,
// and a llama_decode-shaped entry point.  Harness code; depends only on ggml_lite.h (never on the oracle).
#include "llama_lite.h"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "gguf_lite.h"
#include "json_lite.h"
#include "safetensors_lite.h"

#define LLM_ASSERT(x)                                                                           \
    do {                                                                                        \
        if (!(x)) {                                                                             \
            fprintf(stderr, "llama_lite: %s:%d: assertion failed: %s\n", __FILE__, __LINE__, #x); \
            abort();                                                                            \
        }                                                                                       \
    } while (0)

// ---------------------------------------------------------------------------------------------- utilities
static uint16_t f32_to_f16(float f) {  // IEEE binary16, round-to-nearest-even
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t) ((x >> 16) & 0x8000);
    const uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) return (uint16_t) (sign | 0x7C00 | (ax > 0x7F800000u ? 0x200 : 0));
    if (ax >= 0x477FF000u) return (uint16_t) (sign | 0x7C00);
    if (ax < 0x33000001u) return sign;
    const int32_t e = (int32_t) (ax >> 23) - 127;
    uint32_t man = (ax & 0x7FFFFFu) | 0x800000u, shift = 13, base = 0;
    if (e < -14) shift = (uint32_t) (13 + (-14 - e));
    else { base = (uint32_t) (e + 15) << 10; man &= 0x7FFFFFu; }
    const uint32_t halfway = 1u << (shift - 1), rem = man & ((1u << shift) - 1);
    uint32_t q = man >> shift;
    if (rem > halfway || (rem == halfway && (q & 1))) q++;
    return (uint16_t) (sign | (base + q));
}

static inline uint64_t splitmix64(uint64_t & s) {
    uint64_t z = (s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static inline float u01(uint64_t r) { return (float) ((r >> 40) * (1.0 / 16777216.0)); }

static double now_us() {
    return std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

// ------------------------------------------------------------------------------ synthetic quant blocks
// Blocks are sampled directly in the packed domain (SURVEY.md §8d "Synthetic inputs"): quants uniform, 6-bit
// scales uniform with mins tied to scales so that dequantised weights are ~zero-mean with std ~ s/sqrt(K).
// Every block is a pure function of (seed, tensor id, GLOBAL row, GLOBAL block-in-row) so that a
// tensor-parallel shard generates exactly the bytes the unsharded model holds at the same coordinates.
static void synth_block(ggml_type type, uint64_t key, int64_t K, float wscale, uint8_t * out) {
    uint64_t s = key;
    const float scale = wscale * (0.5f + u01(splitmix64(s)));  // s in U(0.5, 1.5) x per-tensor gain
    const float rk = 1.0f / sqrtf((float) K);
    auto fill = [&](uint8_t * p, size_t n) {
        size_t i = 0;
        for (; i + 8 <= n; i += 8) {
            uint64_t r = splitmix64(s);
            memcpy(p + i, &r, 8);
        }
        if (i < n) {
            uint64_t r = splitmix64(s);
            memcpy(p + i, &r, n - i);
        }
    };
    switch (type) {
        case GGML_TYPE_Q8_0: {
            block_q8_0 * b = (block_q8_0 *) out;
            fill((uint8_t *) b->qs, 32);
            for (int i = 0; i < 32; ++i) if (b->qs[i] == -128) b->qs[i] = -127;
            b->d = f32_to_f16(scale * rk / 73.0f);
        } break;
        case GGML_TYPE_Q4_K:
        case GGML_TYPE_Q5_K: {
            uint8_t * p = out;
            uint8_t sc[8], mn[8];
            uint64_t r = splitmix64(s), r2 = splitmix64(s);
            for (int j = 0; j < 8; ++j) {
                sc[j] = (uint8_t) (8 + ((r >> (8 * j)) & 0xFF) % 56);
                int m = (int) sc[j] + (int) ((r2 >> (8 * j)) & 0xFF) % 9 - 4;
                mn[j] = (uint8_t) std::min(63, std::max(0, m));
            }
            const bool q5 = type == GGML_TYPE_Q5_K;
            const float qmean = q5 ? 15.5f : 7.5f, qstd = q5 ? 9.2f : 4.6f;
            const float d = scale * rk / (36.0f * qstd);
            const uint16_t hd = f32_to_f16(d), hm = f32_to_f16(d * qmean);
            memcpy(p, &hd, 2);
            memcpy(p + 2, &hm, 2);
            uint8_t * q = p + 4;
            for (int j = 0; j < 4; ++j) {
                q[j] = (uint8_t) ((sc[j] & 63) | ((sc[j + 4] >> 4) << 6));
                q[j + 4] = (uint8_t) ((mn[j] & 63) | ((mn[j + 4] >> 4) << 6));
                q[j + 8] = (uint8_t) ((sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4));
            }
            fill(p + 16, q5 ? 32 + 128 : 128);
        } break;
        case GGML_TYPE_Q6_K: {
            block_q6_K * b = (block_q6_K *) out;
            fill(b->ql, 128 + 64);
            uint64_t r = splitmix64(s), r2 = splitmix64(s);
            for (int j = 0; j < 16; ++j) {
                uint64_t rr = j < 8 ? r : r2;
                int v = 16 + (int) ((rr >> (8 * (j & 7))) & 0x7F) % 112;  // 16..127
                if ((rr >> (8 * (j & 7) + 7)) & 1) v = -v;
                b->scales[j] = (int8_t) v;
            }
            b->d = f32_to_f16(scale * rk / (70.0f * 18.5f));
        } break;
        default: LLM_ASSERT(!"synth_block: unsupported type");
    }
}

// f16 -> f32 (harness-side: the tied output rows below are re-encoded from token_embd's dequantised values)
static float f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t) (h & 0x8000) << 16, e = (h >> 10) & 31, man = h & 0x3FF;
    uint32_t x;
    if (e == 0) {
        if (!man) x = sign;
        else {
            int sh = 0;
            uint32_t m = man;
            while (!(m & 0x400)) { m <<= 1; ++sh; }
            x = sign | (uint32_t) (127 - 15 - sh + 1) << 23 | (m & 0x3FF) << 13;
        }
    } else if (e == 31) x = sign | 0x7F800000u | man << 13;
    else x = sign | (e + 112) << 23 | man << 13;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

// the 256 values a synthetic K-quant super-block stands for (block layouts: SURVEY.md Appendix A.1 / A.2)
static void block_values(ggml_type type, const uint8_t * p, float * y) {
    auto scale_min = [](int j, const uint8_t * q, int & sc, int & mn) {
        if (j < 4) { sc = q[j] & 63; mn = q[j + 4] & 63; }
        else { sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4); mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4); }
    };
    switch (type) {
        case GGML_TYPE_Q4_K:
        case GGML_TYPE_Q5_K: {
            const bool q5 = type == GGML_TYPE_Q5_K;
            uint16_t hd, hm;
            memcpy(&hd, p, 2);
            memcpy(&hm, p + 2, 2);
            const float d = f16_to_f32(hd), dmin = f16_to_f32(hm);
            const uint8_t * scales = p + 4, * qh = p + 16, * ql = p + (q5 ? 16 + 32 : 16);
            for (int j = 0; j < 4; ++j) {
                int s1, m1, s2, m2;
                scale_min(2 * j, scales, s1, m1);
                scale_min(2 * j + 1, scales, s2, m2);
                for (int l = 0; l < 32; ++l) {
                    const int lo = (ql[32 * j + l] & 0xF) + (q5 && (qh[l] >> (2 * j) & 1) ? 16 : 0);
                    const int hi = (ql[32 * j + l] >> 4) + (q5 && (qh[l] >> (2 * j + 1) & 1) ? 16 : 0);
                    y[64 * j + l] = d * (float) s1 * (float) lo - dmin * (float) m1;
                    y[64 * j + 32 + l] = d * (float) s2 * (float) hi - dmin * (float) m2;
                }
            }
        } break;
        case GGML_TYPE_Q6_K: {
            const block_q6_K * b = (const block_q6_K *) p;
            const float d = f16_to_f32(b->d);
            for (int n = 0; n < 2; ++n) {
                const uint8_t * ql = b->ql + 64 * n, * qh = b->qh + 32 * n;
                const int8_t * sc = b->scales + 8 * n;
                for (int l = 0; l < 32; ++l) {
                    const int is = l / 16;
                    const int q1 = (int) ((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32, q2 = (int) ((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                    const int q3 = (int) ((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32, q4 = (int) ((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                    y[128 * n + l] = d * (float) sc[is] * (float) q1;
                    y[128 * n + l + 32] = d * (float) sc[is + 2] * (float) q2;
                    y[128 * n + l + 64] = d * (float) sc[is + 4] * (float) q3;
                    y[128 * n + l + 96] = d * (float) sc[is + 6] * (float) q4;
                }
            }
        } break;
        default: LLM_ASSERT(!"block_values: unsupported type");
    }
}

// 256 values -> one Q6_K super-block (a plain absmax encoder: any valid block will do for a synthetic weight set — this is the model
// generator, not a restatement of ggml's quantize_row_q6_K)
static void pack_q6_K(const float * x, uint8_t * out) {
    block_q6_K * b = (block_q6_K *) out;
    float sub[16], smax = 0.0f;
    for (int j = 0; j < 16; ++j) {
        float a = 0.0f;
        for (int l = 0; l < 16; ++l) a = std::max(a, fabsf(x[16 * j + l]));
        sub[j] = a / 31.0f;
        smax = std::max(smax, sub[j]);
    }
    memset(b, 0, sizeof(*b));
    if (smax == 0.0f) return;
    const float d = f16_to_f32(f32_to_f16(smax / 127.0f));
    b->d = f32_to_f16(smax / 127.0f);
    int q[256];
    for (int j = 0; j < 16; ++j) {
        const int sc = std::max(1, std::min(127, (int) lrintf(sub[j] / d)));
        b->scales[j] = (int8_t) sc;
        for (int l = 0; l < 16; ++l) q[16 * j + l] = std::max(-32, std::min(31, (int) lrintf(x[16 * j + l] / (d * (float) sc)))) + 32;
    }
    for (int n = 0; n < 2; ++n)
        for (int l = 0; l < 32; ++l) {
            const int q1 = q[128 * n + l], q2 = q[128 * n + l + 32], q3 = q[128 * n + l + 64], q4 = q[128 * n + l + 96];
            b->ql[64 * n + l] = (uint8_t) ((q1 & 0xF) | ((q3 & 0xF) << 4));
            b->ql[64 * n + l + 32] = (uint8_t) ((q2 & 0xF) | ((q4 & 0xF) << 4));
            b->qh[32 * n + l] = (uint8_t) ((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
        }
}

struct synth_spec {
    uint64_t seed;
    int tensor_id;
    ggml_type type;
    int64_t K_global;       // full row length (elements)
    int64_t row_off;        // global index of local row 0
    int64_t blk_off;        // global block index (within a row) of local block 0
    int64_t blocks_per_row; // local
    int64_t blocks_per_row_global;
    int64_t n_rows;         // local
    float f32_lo, f32_hi;   // for F32 tensors
    float wscale;           // gain of quantised tensors
    int tie_id = -1;        // >= 0: `tie_eighths` of every 8 blocks repeat the block of tensor tie_id at row (row * 7919 + 13) % tie_rows (llm_hparams::peaked)
    int tie_eighths = 0;
    int64_t tie_rows = 0;
    ggml_type tie_type = GGML_TYPE_F32;  // the tied tensor's block format; when it is not `type`, its values are re-encoded (Q6_K)
    float tie_wscale = 1.0f;             // ... at the tied tensor's own gain, times tie_gain
    float tie_gain = 1.0f;
};

static void synth_rows(const synth_spec & sp, int64_t row0, int64_t row1, uint8_t * dst) {
    const size_t bs = ggml_abi_type_size(sp.type);
    if (sp.type == GGML_TYPE_F32 || sp.type == GGML_TYPE_F16) {
        const int64_t n = sp.blocks_per_row;  // elements per local row
        for (int64_t r = row0; r < row1; ++r) {
            for (int64_t i = 0; i < n; ++i) {
                uint64_t s = sp.seed ^ ((uint64_t) sp.tensor_id * 0xD1B54A32D192ED03ull) ^ ((uint64_t) ((r + sp.row_off) * sp.blocks_per_row_global + i + sp.blk_off) * 0x9E3779B97F4A7C15ull);
                const float v = sp.f32_lo + (sp.f32_hi - sp.f32_lo) * u01(splitmix64(s));
                if (sp.type == GGML_TYPE_F32) memcpy(dst + ((r - row0) * n + i) * 4, &v, 4);
                else { uint16_t h = f32_to_f16(v); memcpy(dst + ((r - row0) * n + i) * 2, &h, 2); }
            }
        }
        return;
    }
    for (int64_t r = row0; r < row1; ++r) {
        for (int64_t b = 0; b < sp.blocks_per_row; ++b) {
            const uint64_t gb = (uint64_t) ((r + sp.row_off) * sp.blocks_per_row_global + b + sp.blk_off);
            uint64_t key = sp.seed ^ ((uint64_t) sp.tensor_id * 0xD1B54A32D192ED03ull) ^ (gb * 0x9E3779B97F4A7C15ull);
            if (sp.tie_id >= 0) {
                uint64_t pick = key ^ 0xA5A5A5A55A5A5A5Aull;
                if ((int) (splitmix64(pick) & 7) < sp.tie_eighths) {
                    const uint64_t tr = (uint64_t) (((r + sp.row_off) * 7919 + 13) % sp.tie_rows);
                    key = sp.seed ^ ((uint64_t) sp.tie_id * 0xD1B54A32D192ED03ull) ^ ((tr * (uint64_t) sp.blocks_per_row_global + (uint64_t) (b + sp.blk_off)) * 0x9E3779B97F4A7C15ull);
                    if (sp.tie_type != sp.type) {  // Q4_K_M / Q5_K_M: token_embd is Q4_K / Q5_K, output.weight Q6_K — the tied block is token_embd's VALUES in Q6_K
                        LLM_ASSERT(sp.type == GGML_TYPE_Q6_K && ggml_abi_blck_size(sp.tie_type) == 256);
                        uint8_t src[256];
                        float v[256];
                        synth_block(sp.tie_type, key, sp.K_global, sp.tie_wscale, src);
                        block_values(sp.tie_type, src, v);
                        for (float & f : v) f *= sp.tie_gain;
                        pack_q6_K(v, dst + (size_t) ((r - row0) * sp.blocks_per_row + b) * bs);
                        continue;
                    }
                }
            }
            synth_block(sp.type, key, sp.K_global, sp.wscale, dst + (size_t) ((r - row0) * sp.blocks_per_row + b) * bs);
        }
    }
}

// ---------------------------------------------------------------------------------------------- presets
extern "C" int llm_preset(const char * name, struct llm_hparams * hp) {
    memset(hp, 0, sizeof(*hp));
    auto set = [&](const char * arch, int L, int E, int H, int HKV, int HD, int FF, int V, int CTX, float base, float eps, int rope, int bias, int ft) {
        snprintf(hp->arch, sizeof(hp->arch), "%s", arch);
        hp->n_layer = L; hp->n_embd = E; hp->n_head = H; hp->n_head_kv = HKV; hp->n_embd_head = HD; hp->n_ff = FF;
        hp->n_vocab = V; hp->n_ctx_train = CTX; hp->rope_freq_base = base; hp->rms_eps = eps; hp->rope_type = rope;
        hp->qkv_bias = bias; hp->ftype = ft;
    };
    std::string n = name;
    // "<preset>-damped": the same architecture and quantisation recipe with the two properties of a TRAINED network that independent random
    // weights lack — small residual branches (gain 0.08 / sqrt(2 n_layer): a flipped 8-bit activation rounding injects 1/127 of a block's range
    // however small the difference that caused it, and with branches of gain 0.25 every later quantiser re-amplifies it; measured on the oracle
    // against itself, Llama-3-8B: logits NMSE 3.1e-4 at gain 1/8, 4.4e-5 at 0.03, 9.9e-6 at 0.01 — scripts/lab/damped_probe.py) and an output matrix
    // tied to the embeddings (one logit far ahead of the rest): the weight sets north_star's 1e-3 / exact-id bar is testable on
    const bool damped = n.size() > 7 && n.compare(n.size() - 7, 7, "-damped") == 0;
    if (damped) {
        n.resize(n.size() - 7);
        if (llm_preset(n.c_str(), hp) != 0) return -1;
        hp->peaked = 3;
        hp->branch_gain = 0.08f / sqrtf(2.0f * (float) hp->n_layer);
        return 0;
    }
    if (n == "tinyllama-1.1b-q8_0") set("llama", 22, 2048, 32, 4, 64, 5632, 32000, 2048, 10000.0f, 1e-5f, 0, 0, LLM_FTYPE_Q8_0);
    else if (n == "tinyllama-1.1b-q8_0-peaked") { set("llama", 22, 2048, 32, 4, 64, 5632, 32000, 2048, 10000.0f, 1e-5f, 0, 0, LLM_FTYPE_Q8_0); hp->peaked = 3; }
    else if (n == "llama3-8b-q4_k_m") set("llama", 32, 4096, 32, 8, 128, 14336, 128256, 8192, 500000.0f, 1e-5f, 0, 0, LLM_FTYPE_Q4_K_M);
    else if (n == "llama3-70b-q4_k_m") { set("llama", 80, 8192, 64, 8, 128, 28672, 128256, 8192, 500000.0f, 1e-5f, 0, 0, LLM_FTYPE_Q4_K_M); hp->attn_v_q5k_70b = 1; }
    else if (n == "qwen2-7b-q5_k_m") set("qwen2", 28, 3584, 28, 4, 128, 18944, 152064, 32768, 1000000.0f, 1e-6f, GGML_ROPE_TYPE_NEOX, 1, LLM_FTYPE_Q5_K_M);
    // shapes of other families a llama-box user brings (round 6): multi-head attention (1 query head per KV head), 3 query heads per KV head on rows of 12 / 32
    // super-blocks, head_dim 64 with 4 query heads per KV head
    else if (n == "llama3-8b-q8_0") set("llama", 32, 4096, 32, 8, 128, 14336, 128256, 8192, 500000.0f, 1e-5f, 0, 0, LLM_FTYPE_Q8_0);
    else if (n == "llama2-7b-q4_k_m") set("llama", 32, 4096, 32, 32, 128, 11008, 32000, 4096, 10000.0f, 1e-5f, 0, 0, LLM_FTYPE_Q4_K_M);
    else if (n == "llama3.2-3b-q4_k_m") set("llama", 28, 3072, 24, 8, 128, 8192, 128256, 8192, 500000.0f, 1e-5f, 0, 0, LLM_FTYPE_Q4_K_M);
    else if (n == "llama3.2-1b-q4_k_m") set("llama", 16, 2048, 32, 8, 64, 8192, 128256, 8192, 500000.0f, 1e-5f, 0, 0, LLM_FTYPE_Q4_K_M);
    else if (n == "test-llama") set("llama", 3, 256, 4, 2, 64, 512, 512, 512, 10000.0f, 1e-5f, 0, 0, LLM_FTYPE_MIXED);
    else if (n == "test-llama-tp") set("llama", 2, 512, 8, 4, 64, 1024, 512, 512, 10000.0f, 1e-5f, 0, 0, LLM_FTYPE_MIXED);
    // four-way tensor split with head_dim 128: 8 heads on 4 KV heads (2 + 1 per rank), wo K slices of 256, ffn_down K slices of 512, 1024 vocab rows per rank
    else if (n == "test-llama-tp4") set("llama", 2, 1024, 8, 4, 128, 2048, 4096, 512, 10000.0f, 1e-5f, 0, 0, LLM_FTYPE_MIXED);
    else if (n == "test-qwen2") set("qwen2", 2, 256, 4, 2, 64, 768, 768, 512, 1000000.0f, 1e-6f, GGML_ROPE_TYPE_NEOX, 1, LLM_FTYPE_MIXED);
    else return -1;
    return 0;
}

// ---------------------------------------------------------------------------------------------- model
struct llm_layer {
    ggml_tensor *attn_norm = nullptr, *wq = nullptr, *wk = nullptr, *wv = nullptr, *wo = nullptr;
    ggml_tensor *bq = nullptr, *bk = nullptr, *bv = nullptr;
    ggml_tensor *ffn_norm = nullptr, *ffn_gate = nullptr, *ffn_up = nullptr, *ffn_down = nullptr;
    // models described layer by layer (llm_layer_cfg): norms behind the sublayers, the attention output gate, the experts and their router
    ggml_tensor *attn_post_norm = nullptr, *ffn_post_norm = nullptr, *attn_gate = nullptr;
    ggml_tensor *ffn_gate_inp = nullptr, *ffn_up_exps = nullptr, *ffn_down_exps = nullptr;
    // ... a learned sink per head, the (r1, r2) of a distance penalty, the token-shift factors, biases of the feed-forward
    ggml_tensor *attn_sink = nullptr, *attn_r12 = nullptr, *shift = nullptr, *ffn_gate_b = nullptr, *ffn_up_b = nullptr, *ffn_down_b = nullptr;
    // ... latent attention: the down projection to (latent, rotated key part), the latent's norm, the per-head expansions (W_uk stored transposed per
    // head, [dk, rank, head]: the query is taken into the latent space instead of the keys out of it), and the table of rotation frequencies
    ggml_tensor *wdkv = nullptr, *dkv_norm = nullptr, *wuk_t = nullptr, *wuv = nullptr, *rope_freq = nullptr;
    // ... mixers with state per sequence: q, k, v as ONE projection (+ bias), the taps of the short convolution behind it, the raw gates of a recurrence ((b, a) of a
    // delta rule, (i, f) of a matrix memory) with their parameters, the weight of the per-head norm behind the recurrence, the output bias; sigmoid attention's (factor,
    // bias) per head; time mixing: the token-shift taps of its five inputs, the (r, k, v, g) projections as one batched matrix, the decay's two small matrices and
    // offset, the bonus, its norm and its output projection; the gate and up projections of the experts as one tensor
    ggml_tensor *wqkv = nullptr, *bqkv = nullptr, *conv = nullptr, *wgates = nullptr, *gate_par = nullptr, *sub_norm = nullptr, *bo = nullptr, *attn_fb = nullptr;
    ggml_tensor *tm_taps = nullptr, *tm_rkvg = nullptr, *tm_w1 = nullptr, *tm_w2 = nullptr, *tm_w0 = nullptr, *tm_u = nullptr, *tm_norm = nullptr, *tm_out = nullptr;
    ggml_tensor *ffn_gate_up_exps = nullptr;
    // ... a query latent in front of the query heads (down projection, its norm); the weights of a per-head norm on queries and keys (one row shared by the heads)
    ggml_tensor *wdq = nullptr, *dq_norm = nullptr, *q_norm = nullptr, *k_norm = nullptr;
    // ... a delta rule with one decay per key channel beside an attention (its own q, k, v as one projection in wqkv / conv; beta; the decay and the output gate through
    // two small matrices each; its output projection) and the norm weights of the two branches' outputs
    ggml_tensor *wbeta = nullptr, *wa1 = nullptr, *wa2 = nullptr, *wg1 = nullptr, *wg2 = nullptr, *wo_r = nullptr, *left_norm = nullptr, *right_norm = nullptr;
    // ... a state-space mixer: the input projection in three parts (gate z, convolved (x, B, C), step sizes), the convolution's bias
    ggml_tensor *ssm_in_z = nullptr, *ssm_in_xbc = nullptr, *ssm_in_dt = nullptr, *conv_b = nullptr;
    // ... a per-layer token input: the layer's part of a second embedding table, a gate on the stream, the projection back and the norm weight
    ggml_tensor *side_embd = nullptr, *side_gate = nullptr, *side_proj = nullptr, *side_norm = nullptr;
};

// one layer of a model whose config lists its layers one by one (sizes and constants may differ from layer to layer)
enum llm_mlp_kind { LLM_MLP_NONE = 0, LLM_MLP_DENSE = 1, LLM_MLP_MOE = 2 };
// (from LLM_MIX_MLSTM on: mixers that keep state per sequence and bring their own output projection)
enum llm_mixer_kind { LLM_MIX_ATTN = 0, LLM_MIX_LATENT = 1, LLM_MIX_MLSTM = 2, LLM_MIX_DELTA = 3, LLM_MIX_SIGMOID_WKV = 4, LLM_MIX_SSD = 5, LLM_MIX_ATTN_DELTA = 6 };
struct llm_layer_cfg {
    int n_head = 0, n_head_kv = 0, dk = 0, dv = 0;  // query heads, key/value heads, per-head query/key size, per-head value size
    int rot_dims = 0;                               // leading dims of every head that are rotated, as neighbouring pairs
    float rot_base = 10000.0f, scale = 1.0f;
    int chunk = 0;                                  // > 0: a position sees only earlier positions with the same floor(pos / chunk)
    bool sink = false;                              // soft-max denominator carries one more term exp(0): a sink without a value
    bool v_mix = false;                             // values are blended with those of the first such layer ...
    float v_lambda = 0.0f;                          // ... v <- (1 - lambda) v + lambda v_first
    bool out_gate = false;                          // heads are multiplied by sigmoid(W_g h) before the output projection
    int mlp = LLM_MLP_NONE, n_ff = 0, n_expert = 0, n_top = 0;
    int mask_id = 0;                                // index into llm_model::mask_rules
    // mechanisms a design may switch on layer by layer
    int mixer = LLM_MIX_ATTN;
    int window = 0, keep_first = 0;                 // window > 0: position i sees j <= i with i - j < window, and besides the first keep_first positions
    bool v_unit = false;                            // every head's value is divided by its root mean square (no weight) before it is cached
    bool dist_pen = false;                          // score -= r1_h ln(1 + r2_h (i - j)) (attn_r12)
    bool sink_learned = false;                      // the sink's score is a learned number per head (attn_sink) instead of 0
    bool gate_heads = false;                        // the output gate is ONE number per head (W_g has `heads` rows) instead of one per value entry
    bool shift = false;                             // token shift: the mixer reads h + (h_prev - h) * shift, h_prev being the previous token's h (sequence state)
    bool parallel = false;                          // x += mixer(norm(x)) + ff(norm(x)) with ONE norm, instead of two normed sublayers in a row
    bool rms = false;                               // norms are x / sqrt(mean(x^2) + eps) * w instead of layer norms
    bool ffn_gated_tanh = false;                    // W_down (gelu_tanh(W_gate h + b) * (W_up h + b)) + b instead of W_down gelu_erf(W_up h)
    bool rot_half = false;                          // rotation pairs are (i, i + dims / 2) instead of neighbours
    int kv_rank = 0, rot_dim = 0;                   // latent attention: size of the cached latent; the rotated part of a query head / the shared rotated key part
    float yarn_factor = 0.0f, yarn_orig = 0.0f, yarn_fast = 32.0f, yarn_slow = 1.0f;  // yarn_factor > 0: frequencies blended with their 1 / factor (rope_freq)
    bool norm_scalar = false;                       // a norm's weight is ONE number in the checkpoint (kept as a full row here)
    int conv_taps = 0;                              // q, k, v pass a short causal convolution over the sequence (the last tap is the token's own)
    float gate_cap = 0.0f;                          // matrix memory: log gates are capped by cap tanh(. / cap)
    bool sigmoid_attn = false;                      // attention weights are sigmoid(score * factor_h + bias_h) per key, not a soft-max
    float softcap = 0.0f;                           // score <- softcap tanh(score / softcap)
    bool qkv_bias = false, out_bias = false;
    int tm_heads = 0, tm_dim = 0, tm_rank = 0;      // time mixing beside the attention (LLM_MIX_SIGMOID_WKV): heads, head size, inner size of the decay's two matrices
    float left_scale = 1.0f, right_scale = 1.0f;    // the two branches' factors in the mixer's sum
    // mixture of experts: scores are a soft-max over ALL experts; the experts form moe_groups equal groups of neighbours of which the moe_keep with the largest
    // maxima may be chosen from; the chosen scores times moe_scale are the weights (not renormalised); experts are W_down (silu(W_gate h) * W_up h)
    bool moe_scores_all = false;
    int moe_groups = 1, moe_keep = 1;
    float moe_scale = 1.0f;
    bool two_norms = false;                         // with `parallel`: x += mixer(norm1(x)) + ff(norm2(x)), two norms of the same x
    bool ffn_relu_sq = false;                       // dense feed-forward W_down relu(W_up h)^2
    bool qk_norm = false;                           // queries and keys are RMS-normed per head with a weight row shared by the heads
    int q_rank = 0;                                 // > 0: queries come through a normed latent of this size
    int kv_from = -1;                               // >= 0: a latent-attention layer without a down projection of its own, reading that layer's cache rows
    int ssm_state = 0, ssm_groups = 1, ssm_norm_groups = 1;  // state-space mixer (LLM_MIX_SSD): state size per head, groups of (B, C), parts of the gated norm; n_head x dv = inner
    int r_head = 0, r_head_kv = 0, r_dk = 0, r_dv = 0, r_rank = 0;  // the delta rule beside an attention (LLM_MIX_ATTN_DELTA): heads, key heads, sizes, inner size of decay / gate
    int side_dim = 0;                               // > 0: the per-layer token input of this many entries
};
// what a layer's positions may see: one attention mask per distinct rule of a model
struct llm_mask_rule {
    int chunk = 0, window = 0, keep_first = 0;
    bool distance = false;  // the mask holds i - j for visible pairs instead of 0 (layers with a distance penalty)
    bool operator==(const llm_mask_rule & o) const { return chunk == o.chunk && window == o.window && keep_first == o.keep_first && distance == o.distance; }
};
// one execution of a layer: a model may run a range of its layers several times in a row with the same weights; every run has its own cache and state
struct llm_run {
    int il = 0;          // the layer whose weights it uses
    int pass = -1;       // >= 0: number of the pass through the repeated range
    bool first = false;  // the first layer of a pass: the stream is re-projected together with the embedding output before it
                         // (or, without a projection, the embedding output is added from the second pass on), and the pass's step vector is added
};

struct tensor_plan {
    std::string name;
    ggml_type type;
    int64_t ne0, ne1;       // LOCAL shape
    int64_t K_global;       // global ne0
    int64_t row_off, k_off; // shard offsets (elements)
    int tensor_id;
    bool rowpar;            // lives in the reducing (row-parallel) buffer type
    float lo, hi;
    float wscale;
    int tie_id = -1, tie_eighths = 0;
    int64_t tie_rows = 0;
    ggml_type tie_type = GGML_TYPE_F32;
    float tie_wscale = 1.0f;
};

struct llm_model {
    llm_hparams hp{};
    int tp_rank = 0, tp_size = 1;
    int n_head_l = 0, n_head_kv_l = 0, n_ff_l = 0, n_vocab_l = 0;
    ggml_context * ctx = nullptr;
    std::vector<ggml_backend_buffer_t> buffers;
    ggml_tensor *tok_embd = nullptr, *output_norm = nullptr, *output = nullptr;
    std::vector<llm_layer> layers;
    uint64_t stream_bytes = 0, total_bytes = 0;
    int n_dev = 1;               // -sm layer: devices the layers are spread over (llm_model_synth_layer_split)
    std::vector<int> layer_dev;  // ... and which of them holds layer il
    // per-layer description (empty for the uniform llama / qwen2 classes)
    std::vector<llm_layer_cfg> lcfg;
    std::vector<llm_mask_rule> mask_rules;  // the distinct visibility rules of the layers ({} = plain causal): one attention mask each
    std::vector<llm_run> runs;           // the order in which layers execute (one entry per layer unless a range repeats)
    float embd_scale = 1.0f, logit_scale = 1.0f;
    // a hashed bigram embedding added to the token embedding: row (prev * mul_prev + cur * mul_cur) mod buckets, row `buckets` for a sequence's first token
    ggml_tensor * bigram = nullptr;
    int bg_buckets = 0, bg_mul_prev = 0, bg_mul_cur = 0;
    // layers [loop_start, loop_stop) run loop_times times in a row; before each pass x <- loop_in [x; embedding output] + loop_step[pass]
    int loop_start = 0, loop_stop = 0, loop_times = 0;
    ggml_tensor *loop_in = nullptr, *loop_step = nullptr;
    bool has_shift = false;              // some layer keeps the previous token's normed input as sequence state
    bool has_seq_state = false;          // some layer keeps convolution inputs / a recurrence's matrices per sequence: the batch is described by (hist, upd, tok, info)
    int hist_rows = 0;                   // the longest look-back of those layers (taps - 1)
    bool has_attn = true;                // some layer attends over the cell cache (else no masks and no cell indices are made)
    ggml_tensor * attn_sinks = nullptr;  // zeros, one per query head: the sink's score
    ggml_type wtype = GGML_TYPE_F32;     // type of the matrices (and the default type of the cache)
    int max_embd_k = 0, max_embd_v = 0;  // widest K / V cache row over the layers
};

static bool use_more_bits(int i, int n) { return i < n / 8 || i >= 7 * n / 8 || (i - n / 8) % 3 == 2; }

static ggml_type pick_type(const llm_hparams & hp, const char * what, int il) {
    const bool more = use_more_bits(il, hp.n_layer);
    const std::string w = what;
    switch (hp.ftype) {
        case LLM_FTYPE_Q8_0: return GGML_TYPE_Q8_0;
        case LLM_FTYPE_Q6_K: return GGML_TYPE_Q6_K;
        case LLM_FTYPE_F16: return GGML_TYPE_F16;
        case LLM_FTYPE_Q4_K_M:
            if (w == "output") return GGML_TYPE_Q6_K;
            if (w == "attn_v") return more ? GGML_TYPE_Q6_K : (hp.attn_v_q5k_70b ? GGML_TYPE_Q5_K : GGML_TYPE_Q4_K);
            if (w == "ffn_down") return more ? GGML_TYPE_Q6_K : GGML_TYPE_Q4_K;
            return GGML_TYPE_Q4_K;
        case LLM_FTYPE_Q5_K_M:
            if (w == "output") return GGML_TYPE_Q6_K;
            if (w == "attn_v" || w == "ffn_down") return more ? GGML_TYPE_Q6_K : GGML_TYPE_Q5_K;
            return GGML_TYPE_Q5_K;
        case LLM_FTYPE_MIXED: {
            static const ggml_type cyc[4] = {GGML_TYPE_Q4_K, GGML_TYPE_Q5_K, GGML_TYPE_Q6_K, GGML_TYPE_Q8_0};
            unsigned h = (unsigned) il * 7u;
            for (char c : w) h = h * 31u + (unsigned char) c;
            return cyc[h % 4];
        }
        default: return GGML_TYPE_Q8_0;
    }
}

static std::vector<tensor_plan> make_plan(const llm_hparams & hp, int tp_rank, int tp_size, bool split_mm = false) {
    std::vector<tensor_plan> plan;
    int id = 0;
    const int64_t E = hp.n_embd, HD = hp.n_embd_head;
    LLM_ASSERT(hp.n_head % tp_size == 0 && hp.n_head_kv % tp_size == 0 && hp.n_ff % tp_size == 0 && hp.n_vocab % tp_size == 0);
    const int64_t nq = (int64_t) hp.n_head * HD, nkv = (int64_t) hp.n_head_kv * HD;
    const int64_t nq_l = nq / tp_size, nkv_l = nkv / tp_size, ff_l = hp.n_ff / tp_size, v_l = hp.n_vocab / tp_size;
    auto add = [&](const std::string & name, ggml_type type, int64_t ne0, int64_t ne1, int64_t Kg, int64_t row_off, int64_t k_off, bool rowpar, float lo = 0, float hi = 0) {
        // residual-branch output projections get a small gain, as in trained transformers: the residual stream stays
        // dominated by its own history, so one-ulp differences are not chaotically amplified layer over layer
        const bool branch_out = name.find("attn_output") != std::string::npos || name.find("ffn_down") != std::string::npos;
        // (llm_hparams::branch_gain: the "-damped" sets use ~1/sqrt(2 n_layer), the depth scaling trained residual networks are initialised with)
        const float bgain = hp.branch_gain > 0.0f ? hp.branch_gain : 0.25f;
        const float gain = name == "token_embd.weight" ? sqrtf((float) hp.n_embd) : (branch_out ? bgain : 1.0f);  // embeddings ~N(0,1)
        plan.push_back({name, type, ne0, ne1, Kg, row_off, k_off, id++, rowpar, lo, hi, gain});
    };
    add("token_embd.weight", pick_type(hp, "token_embd", 0), E, hp.n_vocab, E, 0, 0, false);
    for (int il = 0; il < hp.n_layer; ++il) {
        const std::string p = "blk." + std::to_string(il) + ".";
        add(p + "attn_norm.weight", GGML_TYPE_F32, E, 1, E, 0, 0, false, 0.5f, 1.5f);
        add(p + "attn_q.weight", pick_type(hp, "attn_q", il), E, nq_l, E, tp_rank * nq_l, 0, false);
        add(p + "attn_k.weight", pick_type(hp, "attn_k", il), E, nkv_l, E, tp_rank * nkv_l, 0, false);
        add(p + "attn_v.weight", pick_type(hp, "attn_v", il), E, nkv_l, E, tp_rank * nkv_l, 0, false);
        if (hp.qkv_bias) {
            add(p + "attn_q.bias", GGML_TYPE_F32, nq_l, 1, nq, 0, tp_rank * nq_l, false, -0.1f, 0.1f);
            add(p + "attn_k.bias", GGML_TYPE_F32, nkv_l, 1, nkv, 0, tp_rank * nkv_l, false, -0.1f, 0.1f);
            add(p + "attn_v.bias", GGML_TYPE_F32, nkv_l, 1, nkv, 0, tp_rank * nkv_l, false, -0.1f, 0.1f);
        }
        add(p + "attn_output.weight", pick_type(hp, "attn_output", il), nq_l, E, nq, 0, tp_rank * nq_l, tp_size > 1);
        add(p + "ffn_norm.weight", GGML_TYPE_F32, E, 1, E, 0, 0, false, 0.5f, 1.5f);
        add(p + "ffn_gate.weight", pick_type(hp, "ffn_gate", il), E, ff_l, E, tp_rank * ff_l, 0, false);
        add(p + "ffn_up.weight", pick_type(hp, "ffn_up", il), E, ff_l, E, tp_rank * ff_l, 0, false);
        add(p + "ffn_down.weight", pick_type(hp, "ffn_down", il), ff_l, E, hp.n_ff, 0, tp_rank * ff_l, tp_size > 1);
    }
    add("output_norm.weight", GGML_TYPE_F32, E, 1, E, 0, 0, false, 0.5f, 1.5f);
    add("output.weight", pick_type(hp, "output", 0), E, v_l, E, tp_rank * v_l, 0, false);
    if (hp.peaked > 0) {
        // the tied blocks are token_embd's: byte for byte (up to the gain) when the two tensors share a format, else its values re-encoded as Q6_K
        LLM_ASSERT(ggml_abi_blck_size(plan.back().type) > 1 && (plan.back().type == plan.front().type || (plan.back().type == GGML_TYPE_Q6_K && ggml_abi_blck_size(plan.front().type) == 256)));
        plan.back().tie_type = plan.front().type;
        plan.back().tie_wscale = plan.front().wscale;
        plan.back().tie_id = plan.front().tensor_id;
        plan.back().tie_eighths = std::min(8, hp.peaked);
        plan.back().tie_rows = hp.n_vocab;
    }
    if (split_mm)  // -sm row: llama.cpp allocates the layers' mat-mul weights and the output matrix in the split buffer type, everything else in the main GPU's
        for (auto & t : plan) {
            const bool mm = t.name.find("attn_q.weight") != std::string::npos || t.name.find("attn_k.weight") != std::string::npos || t.name.find("attn_v.weight") != std::string::npos ||
                            t.name.find("attn_output.weight") != std::string::npos || t.name.find("ffn_") != std::string::npos || t.name == "output.weight";
            t.rowpar = mm && t.name.find("norm") == std::string::npos && ggml_abi_blck_size(t.type) > 1;
        }
    for (auto & t : plan) {
        LLM_ASSERT(t.ne0 % ggml_abi_blck_size(t.type) == 0 && t.k_off % ggml_abi_blck_size(t.type) == 0);
    }
    return plan;
}

static synth_spec spec_of(const tensor_plan & t, uint64_t seed) {
    const int64_t blck = ggml_abi_blck_size(t.type);
    synth_spec sp{};
    sp.seed = seed;
    sp.tensor_id = t.tensor_id;
    sp.type = t.type;
    sp.K_global = t.K_global;
    sp.row_off = t.row_off;
    sp.blk_off = t.k_off / blck;
    sp.blocks_per_row = t.ne0 / blck;
    sp.blocks_per_row_global = t.K_global / blck;
    sp.n_rows = t.ne1;
    sp.f32_lo = t.lo;
    sp.f32_hi = t.hi;
    sp.wscale = t.wscale;
    sp.tie_id = t.tie_id;
    sp.tie_eighths = t.tie_eighths;
    sp.tie_rows = t.tie_rows;
    sp.tie_type = t.tie_id >= 0 ? t.tie_type : t.type;
    sp.tie_wscale = t.tie_wscale;
    sp.tie_gain = t.tie_id >= 0 ? t.wscale / t.tie_wscale : 1.0f;
    return sp;
}

static void bind_tensors(llm_model * m) {
    const llm_hparams & hp = m->hp;
    m->tok_embd = ggml_get_tensor(m->ctx, "token_embd.weight");
    m->output_norm = ggml_get_tensor(m->ctx, "output_norm.weight");
    m->output = ggml_get_tensor(m->ctx, "output.weight");
    if (!m->output) m->output = m->tok_embd;  // tied embeddings
    LLM_ASSERT(m->tok_embd && m->output_norm);
    m->layers.resize(hp.n_layer);
    for (int il = 0; il < hp.n_layer; ++il) {
        const std::string p = "blk." + std::to_string(il) + ".";
        auto g = [&](const char * s) { return ggml_get_tensor(m->ctx, (p + s).c_str()); };
        llm_layer & L = m->layers[il];
        L.attn_norm = g("attn_norm.weight"); L.wq = g("attn_q.weight"); L.wk = g("attn_k.weight"); L.wv = g("attn_v.weight");
        L.wo = g("attn_output.weight"); L.bq = g("attn_q.bias"); L.bk = g("attn_k.bias"); L.bv = g("attn_v.bias");
        L.ffn_norm = g("ffn_norm.weight"); L.ffn_gate = g("ffn_gate.weight"); L.ffn_up = g("ffn_up.weight"); L.ffn_down = g("ffn_down.weight");
        LLM_ASSERT(L.attn_norm && L.wq && L.wk && L.wv && L.wo && L.ffn_norm && L.ffn_gate && L.ffn_up && L.ffn_down);
    }
    m->n_head_l = hp.n_head / m->tp_size;
    m->n_head_kv_l = hp.n_head_kv / m->tp_size;
    m->n_ff_l = hp.n_ff / m->tp_size;
    m->n_vocab_l = (int) m->output->ne[1];
    m->stream_bytes = 0;
    m->total_bytes = 0;
    for (ggml_tensor * t = ggml_get_first_tensor(m->ctx); t; t = ggml_get_next_tensor(m->ctx, t)) {
        m->total_bytes += ggml_nbytes(t);
        if (t == m->tok_embd && m->output != m->tok_embd) m->stream_bytes += ggml_row_size(t->type, t->ne[0]);
        else m->stream_bytes += ggml_nbytes(t);
    }
}

static llm_model * model_synth_impl(const struct llm_hparams * hp, uint64_t seed, ggml_backend_buffer_type_t buft, int tp_rank, int tp_size,
                                    ggml_backend_buffer_type_t rowpar_buft, bool split_mm, const std::vector<ggml_backend_buffer_type_t> * layer_bufts = nullptr);
extern "C" struct llm_model * llm_model_synth(const struct llm_hparams * hp, uint64_t seed, ggml_backend_buffer_type_t buft, int tp_rank, int tp_size,
                                              ggml_backend_buffer_type_t rowpar_buft) {
    return model_synth_impl(hp, seed, buft, tp_rank, tp_size, rowpar_buft, false);
}
// -sm row (llama-box/engine_param.hpp:902-916): one process, every mat-mul weight in `split_buft` — what the backend registry's
// "ggml_backend_split_buffer_type" proc address returned for (main_gpu, tensor_split) — and the rest in the main device's buffer type
extern "C" struct llm_model * llm_model_synth_split(const struct llm_hparams * hp, uint64_t seed, ggml_backend_buffer_type_t buft, ggml_backend_buffer_type_t split_buft) {
    return model_synth_impl(hp, seed, buft, 0, 1, split_buft, true);
}
// -sm layer (llama.cpp's default with several devices; llama-box/engine_param.hpp:900-916): device d holds a contiguous range of layers in its own
// buffer type, token_embd goes with layer 0, output_norm / output with the last layer
static int layer_split_device(int il, int n_layer, int n_dev) { return std::min(n_dev - 1, il * n_dev / std::max(1, n_layer)); }
extern "C" struct llm_model * llm_model_synth_layer_split(const struct llm_hparams * hp, uint64_t seed, const ggml_backend_buffer_type_t * bufts, int n_dev) {
    if (n_dev < 1 || n_dev > hp->n_layer) return nullptr;
    std::vector<ggml_backend_buffer_type_t> v(bufts, bufts + n_dev);
    return model_synth_impl(hp, seed, bufts[0], 0, 1, nullptr, false, &v);
}
static llm_model * model_synth_impl(const struct llm_hparams * hp, uint64_t seed, ggml_backend_buffer_type_t buft, int tp_rank, int tp_size,
                                    ggml_backend_buffer_type_t rowpar_buft, bool split_mm, const std::vector<ggml_backend_buffer_type_t> * layer_bufts) {
    llm_model * m = new llm_model();
    m->hp = *hp;
    m->tp_rank = tp_rank;
    m->tp_size = tp_size;
    m->ctx = ggml_init({0, nullptr, true});
    std::vector<tensor_plan> plan = make_plan(*hp, tp_rank, tp_size, split_mm);
    std::vector<ggml_tensor *> ts;
    for (auto & t : plan) {
        ggml_tensor * x = ggml_new_tensor_2d(m->ctx, t.type, t.ne0, t.ne1);
        ggml_set_name(x, t.name.c_str());
        ts.push_back(x);
    }
    // allocation groups: [0] ordinary weights, [1] row-parallel weights (the backend's reducing / split buffer type), or one group per device of a layer split
    std::vector<ggml_backend_buffer_type_t> group_buft;
    std::vector<int> group_of(plan.size(), 0);
    if (layer_bufts) {
        group_buft = *layer_bufts;
        m->n_dev = (int) layer_bufts->size();
        m->layer_dev.resize((size_t) hp->n_layer);
        for (int il = 0; il < hp->n_layer; ++il) m->layer_dev[(size_t) il] = layer_split_device(il, hp->n_layer, m->n_dev);
        for (size_t i = 0; i < plan.size(); ++i) {
            int il = -1;
            if (sscanf(plan[i].name.c_str(), "blk.%d.", &il) == 1) group_of[i] = m->layer_dev[(size_t) il];
            else group_of[i] = plan[i].name == "token_embd.weight" ? 0 : m->n_dev - 1;
        }
    } else {
        group_buft = {buft, rowpar_buft};
        for (size_t i = 0; i < plan.size(); ++i) group_of[i] = (plan[i].rowpar && rowpar_buft) ? 1 : 0;
    }
    {
        std::vector<size_t> total(group_buft.size(), 0), off(group_buft.size(), 0);
        std::vector<ggml_backend_buffer_t> bufs(group_buft.size(), nullptr);
        for (size_t i = 0; i < plan.size(); ++i) {
            const int g = group_of[i];
            const size_t align = ggml_backend_buft_get_alignment(group_buft[(size_t) g]);
            total[(size_t) g] = (total[(size_t) g] + align - 1) / align * align + ggml_backend_buft_get_alloc_size(group_buft[(size_t) g], ts[i]);
        }
        for (size_t g = 0; g < group_buft.size(); ++g) {
            if (!total[g]) continue;
            bufs[g] = ggml_backend_buft_alloc_buffer(group_buft[g], total[g] + ggml_backend_buft_get_alignment(group_buft[g]));
            if (!bufs[g]) {
                fprintf(stderr, "llm_model_synth: failed to allocate %zu bytes of weights\n", total[g]);
                llm_model_free(m);
                return nullptr;
            }
            ggml_backend_buffer_set_usage(bufs[g], GGML_BACKEND_BUFFER_USAGE_WEIGHTS);
            m->buffers.push_back(bufs[g]);
        }
        for (size_t i = 0; i < plan.size(); ++i) {
            const size_t g = (size_t) group_of[i];
            const size_t align = ggml_backend_buft_get_alignment(group_buft[g]);
            ggml_backend_buffer_t bb = bufs[g];
            off[g] = (off[g] + align - 1) / align * align;
            ts[i]->data = (char *) ggml_backend_buffer_get_base(bb) + off[g];
            ts[i]->buffer = bb;
            if (bb->iface.init_tensor && bb->iface.init_tensor(bb, ts[i]) != GGML_STATUS_SUCCESS) {
                fprintf(stderr, "llm_model_synth: init_tensor failed for %s\n", plan[i].name.c_str());
                llm_model_free(m);
                return nullptr;
            }
            off[g] += ggml_backend_buft_get_alloc_size(group_buft[g], ts[i]);
        }
    }
    // generate + upload in chunks of rows, generation multi-threaded (each block is independent)
    const unsigned nthr = std::max(1u, std::min(32u, std::thread::hardware_concurrency()));
    std::vector<uint8_t> stage;
    for (size_t i = 0; i < plan.size(); ++i) {
        const synth_spec sp = spec_of(plan[i], seed);
        const size_t row_bytes = ggml_row_size(plan[i].type, plan[i].ne0);
        // (a split buffer takes whole tensors only, like upstream's: the loader writes a tensor in one call)
        const int64_t rows_per_chunk = (split_mm && plan[i].rowpar) ? plan[i].ne1 : std::max<int64_t>(1, (int64_t) ((64u << 20) / row_bytes));
        for (int64_t r0 = 0; r0 < plan[i].ne1; r0 += rows_per_chunk) {
            const int64_t r1 = std::min<int64_t>(plan[i].ne1, r0 + rows_per_chunk);
            stage.resize((size_t) (r1 - r0) * row_bytes);
            std::vector<std::thread> th;
            const int64_t per = (r1 - r0 + nthr - 1) / nthr;
            for (unsigned t = 0; t < nthr; ++t) {
                const int64_t a = r0 + t * per, b = std::min(r1, a + per);
                if (a >= b) break;
                th.emplace_back([&, a, b]() { synth_rows(sp, a, b, stage.data() + (size_t) (a - r0) * row_bytes); });
            }
            for (auto & x : th) x.join();
            ggml_backend_tensor_set(ts[i], stage.data(), (size_t) r0 * row_bytes, stage.size());
        }
    }
    bind_tensors(m);
    return m;
}

struct gguf_fill_ctx {
    const std::vector<tensor_plan> * plan;
    uint64_t seed;
};
static void gguf_fill(const gguf_tensor_info & ti, void * dst, void * user) {
    gguf_fill_ctx * c = (gguf_fill_ctx *) user;
    for (auto & t : *c->plan) {
        if (t.name == ti.name) {
            synth_rows(spec_of(t, c->seed), 0, t.ne1, (uint8_t *) dst);
            return;
        }
    }
    LLM_ASSERT(!"gguf_fill: unknown tensor");
}

extern "C" int llm_synth_gguf(const struct llm_hparams * hp, uint64_t seed, const char * path) {
    std::vector<tensor_plan> plan = make_plan(*hp, 0, 1);
    gguf_writer w;
    const std::string a = hp->arch;
    w.set_str("general.architecture", a);
    w.set_str("general.name", "synthetic-" + a);
    w.set_u32("general.alignment", 32);
    w.set_u32("general.file_type", (uint32_t) hp->ftype);
    w.set_u32(a + ".block_count", (uint32_t) hp->n_layer);
    w.set_u32(a + ".context_length", (uint32_t) hp->n_ctx_train);
    w.set_u32(a + ".embedding_length", (uint32_t) hp->n_embd);
    w.set_u32(a + ".feed_forward_length", (uint32_t) hp->n_ff);
    w.set_u32(a + ".attention.head_count", (uint32_t) hp->n_head);
    w.set_u32(a + ".attention.head_count_kv", (uint32_t) hp->n_head_kv);
    w.set_f32(a + ".attention.layer_norm_rms_epsilon", hp->rms_eps);
    w.set_f32(a + ".rope.freq_base", hp->rope_freq_base);
    w.set_u32(a + ".rope.dimension_count", (uint32_t) hp->n_embd_head);
    w.set_u32(a + ".vocab_size", (uint32_t) hp->n_vocab);
    w.set_str("tokenizer.ggml.model", "no_vocab");
    for (auto & t : plan) {
        const int64_t ne[2] = {t.ne0, t.ne1};
        w.add_tensor(t.name, t.type, t.ne1 == 1 ? 1 : 2, ne);
    }
    gguf_fill_ctx fc{&plan, seed};
    return w.write(path, gguf_fill, &fc) ? 0 : -1;
}

extern "C" struct llm_model * llm_model_load(const char * path, ggml_backend_buffer_type_t buft) {
    gguf_file * f = gguf_open(path);
    if (!f) return nullptr;
    llm_model * m = new llm_model();
    llm_hparams & hp = m->hp;
    const std::string a = f->get_s("general.architecture", "llama");
    snprintf(hp.arch, sizeof(hp.arch), "%s", a.c_str());
    hp.n_layer = (int) f->get_u(a + ".block_count");
    hp.n_ctx_train = (int) f->get_u(a + ".context_length");
    hp.n_embd = (int) f->get_u(a + ".embedding_length");
    hp.n_ff = (int) f->get_u(a + ".feed_forward_length");
    hp.n_head = (int) f->get_u(a + ".attention.head_count");
    hp.n_head_kv = (int) f->get_u(a + ".attention.head_count_kv", hp.n_head);
    hp.rms_eps = (float) f->get_f(a + ".attention.layer_norm_rms_epsilon", 1e-5);
    hp.rope_freq_base = (float) f->get_f(a + ".rope.freq_base", 10000.0);
    hp.n_embd_head = (int) f->get_u(a + ".rope.dimension_count", hp.n_head ? hp.n_embd / hp.n_head : 0);
    hp.ftype = (int) f->get_u("general.file_type");
    hp.rope_type = a == "qwen2" ? GGML_ROPE_TYPE_NEOX : 0;
    const gguf_tensor_info * te = f->find("token_embd.weight");
    if (!te || hp.n_layer <= 0 || hp.n_embd <= 0 || hp.n_head <= 0) {
        fprintf(stderr, "llm_model_load: %s: missing hyper-parameters or token_embd.weight\n", path);
        delete f;
        delete m;
        return nullptr;
    }
    hp.n_vocab = (int) f->get_u(a + ".vocab_size", (uint64_t) te->ne[1]);
    hp.qkv_bias = f->find("blk.0.attn_q.bias") != nullptr;
    m->ctx = ggml_init({0, nullptr, true});
    for (auto & ti : f->tensors) {
        ggml_tensor * t = ggml_new_tensor(m->ctx, ti.type, ti.n_dims, ti.ne);
        ggml_set_name(t, ti.name.c_str());
    }
    ggml_backend_buffer_t buf = ggml_backend_alloc_ctx_tensors_from_buft(m->ctx, buft);
    if (!buf) {
        fprintf(stderr, "llm_model_load: failed to allocate weights\n");
        delete f;
        llm_model_free(m);
        return nullptr;
    }
    ggml_backend_buffer_set_usage(buf, GGML_BACKEND_BUFFER_USAGE_WEIGHTS);
    m->buffers.push_back(buf);
    for (auto & ti : f->tensors) ggml_backend_tensor_set(ggml_get_tensor(m->ctx, ti.name.c_str()), f->tensor_data(ti), 0, ti.size);
    delete f;
    bind_tensors(m);
    return m;
}

// ---------------------------------------------------------------------------------------------- models from a checkpoint folder
// config.json names the architecture and lists the layers; model.safetensors holds bf16 matrices stored [out, in].  The tensors are
// re-named to the framework's own scheme (token_embd, blk.N.attn_q, ...); the experts of a layer are stacked into one 3-d tensor per
// projection, the form MUL_MAT_ID reads.
static float bf16_to_f32(uint16_t h) {
    const uint32_t x = (uint32_t) h << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}
static uint16_t f32_to_bf16(float f) {  // round to nearest even
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t) ((x >> 16) | 0x40);
    return (uint16_t) ((x + 0x7FFFu + ((x >> 16) & 1u)) >> 16);
}

struct dir_tensor {               // one framework tensor and where its values come from
    std::string name;             // framework name
    ggml_type type;
    int64_t ne[3];
    std::vector<std::string> src; // checkpoint tensors, stacked along the last dim (one entry unless experts)
    float synth_gain;             // random weights: N(0, gain^2 / ne0); < 0: 1 + 0.1 N(0, 1) (norm weights)
    bool head_transpose = false;  // the checkpoint tensor is [ne2 * ne0, ne1] (heads x rows, columns): kept as ne2 matrices [ne0, ne1] with the ROWS along dim 0
    std::vector<float> values;    // not from the checkpoint: computed by the loader (f32 tensors)
    float synth_lo = 0.0f, synth_hi = 0.0f;  // random weights: uniform in [lo, hi) when hi > lo (shift factors, penalties)
    bool broadcast = false;       // the checkpoint holds ONE number: every entry of the tensor gets it (a norm with a scalar weight)
    bool mix_taps = false;        // src are token-shift factors mu [ne1] each: kept as 2-tap convolution weights (mu for the previous token, 1 - mu for the token's own), [2, ne1, n_src]
    bool one_plus = false;        // a norm weight stored around zero: 1 is added to every entry (f32 tensors)
    int64_t row0 = -1;            // >= 0: the ONE source is [rows, ne0] and rows row0 .. row0 + ne1 - 1 of it are taken (a projection stored as one matrix, kept in parts)
    int64_t col0 = -1;            // >= 0: the ONE source is [ne1, columns] and columns col0 .. col0 + ne0 - 1 of every row are taken (a layer's part of a shared table)
};

// the visibility rule of a layer gets a mask of its own unless another layer has the same
static int mask_rule_id(llm_model * m, const llm_mask_rule & r) {
    size_t k = 0;
    while (k < m->mask_rules.size() && !(m->mask_rules[k] == r)) ++k;
    if (k == m->mask_rules.size()) m->mask_rules.push_back(r);
    return (int) k;
}

static bool parse_nigozen_config(const json_value & cfg, llm_model * m, std::string & err) {
    llm_hparams & hp = m->hp;
    snprintf(hp.arch, sizeof(hp.arch), "nigozen");
    const json_value * layers = cfg.get("layers");
    if (!layers || layers->kind != json_value::ARR || layers->arr.empty()) { err = "config: no layers"; return false; }
    const json_value * v;
    hp.n_embd = (v = cfg.get("width")) ? (int) v->number(0) : 0;
    hp.n_vocab = (v = cfg.get("vocab")) ? (int) v->number(0) : 0;
    hp.rms_eps = (v = cfg.path("norm", "eps")) ? (float) v->number(1e-5) : 1e-5f;
    m->embd_scale = (v = cfg.path("embedding", "scale")) ? (float) v->number(1.0) : 1.0f;
    hp.n_layer = (int) layers->arr.size();
    hp.n_ctx_train = 1 << 20;
    if (hp.n_embd <= 0 || hp.n_vocab <= 0) { err = "config: width / vocab missing"; return false; }
    m->lcfg.resize((size_t) hp.n_layer);
    for (int il = 0; il < hp.n_layer; ++il) {
        const json_value & L = layers->arr[(size_t) il];
        llm_layer_cfg & c = m->lcfg[(size_t) il];
        const json_value * type = L.get("type");
        if (!type || type->kind != json_value::STR || type->str != "attention") { err = "config: layer " + std::to_string(il) + ": unknown mixer type"; return false; }
        const json_value * mx = L.get("mixer");
        if (!mx || mx->kind != json_value::OBJ) { err = "config: layer without a mixer"; return false; }
        auto num = [&](const json_value * o, const char * k0, const char * k1, double d) { const json_value * x = o->path(k0, k1); return x ? x->number(d) : d; };
        c.n_head = (int) num(mx, "heads", nullptr, 0);
        c.n_head_kv = (int) num(mx, "kv_heads", nullptr, c.n_head);
        c.dk = (int) num(mx, "dim", nullptr, 0);
        c.dv = (int) num(mx, "vdim", nullptr, c.dk);
        c.rot_dims = (int) num(mx, "rot", "dims", 0);
        c.rot_base = (float) num(mx, "rot", "base", 10000.0);
        c.scale = (float) num(mx, "scale", nullptr, c.dk > 0 ? 1.0 / sqrt((double) c.dk) : 1.0);
        c.chunk = (int) num(mx, "mask", "size", 0);
        c.v_mix = num(mx, "v_mix", nullptr, 0) != 0;
        c.sink = true;      // the design's soft-max always carries the sink ...
        c.out_gate = true;  // ... and its heads always pass the sigmoid gate
        if (c.n_head <= 0 || c.n_head_kv <= 0 || c.n_head % c.n_head_kv || c.dk <= 0 || c.dv <= 0 || c.rot_dims < 0 || c.rot_dims > c.dk || (c.rot_dims & 1) || c.chunk < 0) {
            err = "config: layer " + std::to_string(il) + ": inconsistent attention sizes";
            return false;
        }
        const json_value * ml = L.path("mlp");
        if (ml) {
            const json_value * kind = ml->get("kind");
            if (kind && kind->kind == json_value::STR && kind->str == "dense") {
                c.mlp = LLM_MLP_DENSE;
                c.n_ff = (int) num(ml, "ff", nullptr, 0);
            } else if (kind && kind->kind == json_value::STR && kind->str == "moe") {
                c.mlp = LLM_MLP_MOE;
                c.n_ff = (int) num(ml, "expert", "ff", 0);
                c.n_expert = (int) num(ml, "router", "experts", 0);
                c.n_top = (int) num(ml, "router", "top", 0);
                if (c.n_expert <= 0 || c.n_top <= 0 || c.n_top > c.n_expert) { err = "config: layer " + std::to_string(il) + ": inconsistent router"; return false; }
            } else { err = "config: layer " + std::to_string(il) + ": unknown mlp kind"; return false; }
            if (c.n_ff <= 0) { err = "config: layer " + std::to_string(il) + ": ff missing"; return false; }
        }
        llm_mask_rule rule;
        rule.chunk = c.chunk;
        c.mask_id = mask_rule_id(m, rule);
        m->max_embd_k = std::max(m->max_embd_k, c.n_head_kv * c.dk);
        m->max_embd_v = std::max(m->max_embd_v, c.n_head_kv * c.dv);
    }
    // the uniform fields describe layer 0 (informational for per-layer models)
    hp.n_head = m->lcfg[0].n_head; hp.n_head_kv = m->lcfg[0].n_head_kv; hp.n_embd_head = m->lcfg[0].dk; hp.n_ff = m->lcfg[0].n_ff;
    hp.rope_freq_base = m->lcfg[0].rot_base;
    for (int il = 0; il < hp.n_layer; ++il) m->runs.push_back({il, -1, false});
    return true;
}

// Zigipel: every layer is x += mixer(shift(h)) + ff(h) with h = rms_norm(x) (one norm, both sublayers read it; the mixer's copy is blended with the previous
// token's h).  Mixers: grouped-query attention without rotation (unit-rms values, a logarithmic distance penalty, a sliding window that also keeps the first
// tokens, a learned sink, one sigmoid gate per head), or latent attention (keys and values expanded from a cached normed latent, one rotated key part shared
// by the heads, rotate-half layout with YaRN-blended frequencies, sliding window, learned sink).  Gated tanh-GELU feed-forward with biases.  A hashed bigram
// embedding is added to the token embedding; a range of layers repeats; the output matrix is its own tensor and the logits are scaled.
static bool parse_zigipel_config(const json_value & cfg, llm_model * m, std::string & err) {
    llm_hparams & hp = m->hp;
    snprintf(hp.arch, sizeof(hp.arch), "zigipel");
    const json_value * layers = cfg.get("layers");
    if (!layers || layers->kind != json_value::ARR || layers->arr.empty()) { err = "config: no layers"; return false; }
    const json_value * v;
    hp.n_embd = (v = cfg.get("width")) ? (int) v->number(0) : 0;
    hp.n_vocab = (v = cfg.get("vocab")) ? (int) v->number(0) : 0;
    hp.rms_eps = (v = cfg.path("norm", "eps")) ? (float) v->number(1e-5) : 1e-5f;
    m->logit_scale = (v = cfg.get("logit_scale")) ? (float) v->number(1.0) : 1.0f;
    hp.n_layer = (int) layers->arr.size();
    hp.n_ctx_train = 1 << 20;
    if (hp.n_embd <= 0 || hp.n_vocab <= 0) { err = "config: width / vocab missing"; return false; }
    auto num = [&](const json_value * o, const char * k0, const char * k1, double d) { const json_value * x = o->path(k0, k1); return x ? x->number(d) : d; };
    if (const json_value * bg = cfg.path("embedding", "bigram")) {
        m->bg_buckets = (int) num(bg, "buckets", nullptr, 0);
        m->bg_mul_prev = (int) num(bg, "mul_prev", nullptr, 0);
        m->bg_mul_cur = (int) num(bg, "mul_cur", nullptr, 0);
        if (m->bg_buckets <= 0) { err = "config: bigram embedding without buckets"; return false; }
    }
    if (const json_value * lp = cfg.get("loop")) {
        m->loop_start = (int) num(lp, "start", nullptr, 0);
        m->loop_stop = (int) num(lp, "stop", nullptr, 0);
        m->loop_times = (int) num(lp, "times", nullptr, 1);
        if (m->loop_start < 0 || m->loop_stop > hp.n_layer || m->loop_start >= m->loop_stop || m->loop_times < 1) { err = "config: inconsistent loop"; return false; }
    }
    m->lcfg.resize((size_t) hp.n_layer);
    for (int il = 0; il < hp.n_layer; ++il) {
        const json_value & L = layers->arr[(size_t) il];
        llm_layer_cfg & c = m->lcfg[(size_t) il];
        const std::string lname = "config: layer " + std::to_string(il);
        const json_value * type = L.get("type");
        const json_value * mx = L.get("mixer");
        if (!type || type->kind != json_value::STR || !mx || mx->kind != json_value::OBJ) { err = lname + ": no mixer"; return false; }
        c.parallel = c.rms = c.shift = c.sink_learned = true;
        c.sink = true;
        c.n_head = (int) num(mx, "heads", nullptr, 0);
        c.dk = (int) num(mx, "dim", nullptr, 0);
        c.dv = (int) num(mx, "vdim", nullptr, c.dk);
        c.scale = (float) num(mx, "scale", nullptr, c.dk > 0 ? 1.0 / sqrt((double) c.dk) : 1.0);
        c.window = (int) num(mx, "mask", "size", 0);
        c.rot_dims = 0;
        if (type->str == "attention") {
            c.mixer = LLM_MIX_ATTN;
            c.n_head_kv = (int) num(mx, "kv_heads", nullptr, c.n_head);
            c.keep_first = (int) num(mx, "mask", "keep_first", 0);
            c.v_unit = c.dist_pen = c.out_gate = c.gate_heads = true;
            if (c.n_head <= 0 || c.n_head_kv <= 0 || c.n_head % c.n_head_kv || c.dk <= 0 || c.dv <= 0 || c.window < 0 || c.keep_first < 0) { err = lname + ": inconsistent attention sizes"; return false; }
            m->max_embd_k = std::max(m->max_embd_k, c.n_head_kv * c.dk);
            m->max_embd_v = std::max(m->max_embd_v, c.n_head_kv * c.dv);
        } else if (type->str == "latent_attention") {
            c.mixer = LLM_MIX_LATENT;
            c.n_head_kv = 1;
            c.kv_rank = (int) num(mx, "kv_rank", nullptr, 0);
            c.rot_dim = (int) num(mx, "rot_dim", nullptr, 0);
            c.rot_dims = c.rot_dim;  // the rotated vector is the rot_dim part of a head
            c.rot_half = true;
            c.rot_base = (float) num(mx, "rot", "base", 10000.0);
            if (const json_value * sc = mx->path("rot", "scaling")) {
                c.yarn_factor = (float) num(sc, "factor", nullptr, 1.0);
                c.yarn_orig = (float) num(sc, "original", nullptr, 0.0);
                c.yarn_fast = (float) num(sc, "fast", nullptr, 32.0);
                c.yarn_slow = (float) num(sc, "slow", nullptr, 1.0);
                if (c.yarn_factor <= 0.0f || c.yarn_orig <= 0.0f) { err = lname + ": inconsistent rotary scaling"; return false; }
            }
            if (c.n_head <= 0 || c.dk <= 0 || c.dv <= 0 || c.kv_rank <= 0 || c.rot_dim < 0 || (c.rot_dim & 1) || c.window < 0) { err = lname + ": inconsistent latent attention sizes"; return false; }
            m->max_embd_k = std::max(m->max_embd_k, c.kv_rank + c.rot_dim);
        } else { err = lname + ": unknown mixer type"; return false; }
        const json_value * ml = L.path("mlp");
        if (ml && ml->kind == json_value::OBJ) {
            const json_value * kind = ml->get("kind");
            if (!kind || kind->kind != json_value::STR || kind->str != "dense") { err = lname + ": unknown mlp kind"; return false; }
            c.mlp = LLM_MLP_DENSE;
            c.ffn_gated_tanh = true;
            c.n_ff = (int) num(ml, "ff", nullptr, 0);
            if (c.n_ff <= 0) { err = lname + ": ff missing"; return false; }
        }
        llm_mask_rule rule;
        rule.window = c.window;
        rule.keep_first = c.window > 0 ? c.keep_first : 0;
        rule.distance = c.dist_pen;
        c.mask_id = mask_rule_id(m, rule);
    }
    m->has_shift = true;
    hp.n_head = m->lcfg[0].n_head; hp.n_head_kv = m->lcfg[0].n_head_kv; hp.n_embd_head = m->lcfg[0].dk; hp.n_ff = m->lcfg[0].n_ff;
    hp.rope_freq_base = m->lcfg[0].rot_base;
    // the order of execution: layers before the repeated range, the range `times` times, the rest
    for (int il = 0; il < (m->loop_times > 0 ? m->loop_start : hp.n_layer); ++il) m->runs.push_back({il, -1, false});
    if (m->loop_times > 0) {
        for (int t = 0; t < m->loop_times; ++t)
            for (int il = m->loop_start; il < m->loop_stop; ++il) m->runs.push_back({il, t, il == m->loop_start});
        for (int il = m->loop_stop; il < hp.n_layer; ++il) m->runs.push_back({il, -1, false});
    }
    return true;
}


// Rarelorn: pre-norm layers x += mixer(norm1(x)); x += ff(norm2(x)) with scalar-weight RMS norms.  Mixers, all with state per sequence: a matrix memory with
// exponential gates (mlstm), a gated delta rule behind short convolutions (delta), and windowed sigmoid attention (biases, short convolutions, partial rotate-half
// positions, soft-capped scores) side by side with RWKV-style time mixing (parallel).  Feed-forward: experts chosen by a soft-max over all of them, confined to the
// best groups.  A range of layers repeats; from the second pass on the embedding output is added, and a step vector every pass.
static bool parse_rarelorn_config(const json_value & cfg, const st_file * file, llm_model * m, std::string & err) {
    llm_hparams & hp = m->hp;
    snprintf(hp.arch, sizeof(hp.arch), "rarelorn");
    const json_value * layers = cfg.get("layers");
    if (!layers || layers->kind != json_value::ARR || layers->arr.empty()) { err = "config: no layers"; return false; }
    const json_value * v;
    hp.n_embd = (v = cfg.get("width")) ? (int) v->number(0) : 0;
    hp.n_vocab = (v = cfg.get("vocab")) ? (int) v->number(0) : 0;
    hp.rms_eps = (v = cfg.path("norm", "eps")) ? (float) v->number(1e-5) : 1e-5f;
    hp.n_layer = (int) layers->arr.size();
    hp.n_ctx_train = 1 << 20;
    if (hp.n_embd <= 0 || hp.n_vocab <= 0) { err = "config: width / vocab missing"; return false; }
    auto num = [&](const json_value * o, const char * k0, const char * k1, double d) { const json_value * x = o->path(k0, k1); return x ? x->number(d) : d; };
    if (const json_value * lp = cfg.get("loop")) {
        if (lp->kind == json_value::OBJ) {
            m->loop_start = (int) num(lp, "start", nullptr, 0);
            m->loop_stop = (int) num(lp, "stop", nullptr, 0);
            m->loop_times = (int) num(lp, "times", nullptr, 1);
            if (m->loop_start < 0 || m->loop_stop > hp.n_layer || m->loop_start >= m->loop_stop || m->loop_times < 1) { err = "config: inconsistent loop"; return false; }
        }
    }
    m->lcfg.resize((size_t) hp.n_layer);
    m->has_attn = false;
    m->has_seq_state = true;
    m->hist_rows = 0;
    for (int il = 0; il < hp.n_layer; ++il) {
        const json_value & L = layers->arr[(size_t) il];
        llm_layer_cfg & c = m->lcfg[(size_t) il];
        const std::string lname = "config: layer " + std::to_string(il);
        const json_value * type = L.get("type");
        const json_value * mx = L.get("mixer");
        if (!type || type->kind != json_value::STR || !mx || mx->kind != json_value::OBJ) { err = lname + ": no mixer"; return false; }
        c.rms = c.norm_scalar = true;
        if (type->str == "mlstm") {
            c.mixer = LLM_MIX_MLSTM;
            c.n_head = c.n_head_kv = (int) num(mx, "heads", nullptr, 0);
            c.dk = (int) num(mx, "dim", nullptr, 0);
            c.dv = (int) num(mx, "vdim", nullptr, c.dk);
            c.gate_cap = (float) num(mx, "gate_cap", nullptr, 15.0);
            if (c.n_head <= 0 || c.dk <= 0 || c.dv <= 0 || c.gate_cap <= 0.0f) { err = lname + ": inconsistent matrix-memory sizes"; return false; }
        } else if (type->str == "delta") {
            c.mixer = LLM_MIX_DELTA;
            c.n_head = (int) num(mx, "heads", nullptr, 0);
            c.n_head_kv = (int) num(mx, "kv_heads", nullptr, c.n_head);
            c.dk = (int) num(mx, "dim", nullptr, 0);
            c.dv = (int) num(mx, "vdim", nullptr, c.dk);
            c.conv_taps = (int) num(mx, "conv", nullptr, 1);
            if (c.n_head <= 0 || c.n_head_kv <= 0 || c.n_head % c.n_head_kv || c.dk <= 0 || c.dv <= 0 || c.conv_taps < 1 || c.conv_taps > 16) { err = lname + ": inconsistent delta-rule sizes"; return false; }
        } else if (type->str == "parallel") {
            c.mixer = LLM_MIX_SIGMOID_WKV;
            const json_value * lf = mx->get("left"), * rt = mx->get("right");
            if (!lf || lf->kind != json_value::OBJ || !rt || rt->kind != json_value::OBJ) { err = lname + ": a parallel mixer needs left and right"; return false; }
            c.n_head = (int) num(lf, "heads", nullptr, 0);
            c.n_head_kv = (int) num(lf, "kv_heads", nullptr, c.n_head);
            c.dk = (int) num(lf, "dim", nullptr, 0);
            c.dv = (int) num(lf, "vdim", nullptr, c.dk);
            c.conv_taps = (int) num(lf, "conv", nullptr, 1);
            c.window = (int) num(lf, "mask", "size", 0);
            c.rot_dims = (int) num(lf, "rot", "dims", 0);
            c.rot_base = (float) num(lf, "rot", "base", 10000.0);
            c.rot_half = true;
            c.scale = (float) num(lf, "scale", nullptr, c.dk > 0 ? 1.0 / sqrt((double) c.dk) : 1.0);
            c.softcap = (float) num(lf, "softcap", nullptr, 0.0);
            c.sigmoid_attn = c.qkv_bias = c.out_bias = true;
            c.tm_heads = (int) num(rt, "heads", nullptr, 0);
            c.tm_dim = (int) num(rt, "dim", nullptr, 0);
            c.tm_rank = (int) num(rt, "rank", nullptr, 16);  // (a checkpoint's w1 gives it)
            if (file) {
                const st_tensor * w1 = file->find("l" + std::to_string(il) + ".mix.right.w1");
                if (!w1 || w1->shape.size() != 2) { err = lname + ": no right.w1 in the checkpoint"; return false; }
                c.tm_rank = (int) w1->shape[0];
            }
            c.left_scale = (float) num(mx, "left_scale", nullptr, 1.0);
            c.right_scale = (float) num(mx, "right_scale", nullptr, 1.0);
            if (c.n_head <= 0 || c.n_head_kv <= 0 || c.n_head % c.n_head_kv || c.dk <= 0 || c.dv <= 0 || c.conv_taps < 1 || c.conv_taps > 16 || c.window < 0 || c.rot_dims < 0 ||
                c.rot_dims > c.dk || (c.rot_dims & 1) || c.softcap < 0.0f || c.tm_heads <= 0 || c.tm_dim <= 0 || c.tm_rank <= 0) { err = lname + ": inconsistent parallel-mixer sizes"; return false; }
            m->has_attn = true;
            m->hist_rows = std::max(m->hist_rows, 1);  // (the time mixing's token shift looks one token back)
            m->max_embd_k = std::max(m->max_embd_k, c.n_head_kv * c.dk);
            m->max_embd_v = std::max(m->max_embd_v, c.n_head_kv * c.dv);
            llm_mask_rule rule;
            rule.window = c.window;
            c.mask_id = mask_rule_id(m, rule);
        } else { err = lname + ": unknown mixer type"; return false; }
        m->hist_rows = std::max(m->hist_rows, c.conv_taps - 1);
        const json_value * ml = L.path("mlp");
        if (ml && ml->kind == json_value::OBJ) {
            const json_value * kind = ml->get("kind");
            if (!kind || kind->kind != json_value::STR || kind->str != "moe") { err = lname + ": unknown mlp kind"; return false; }
            c.mlp = LLM_MLP_MOE;
            c.moe_scores_all = true;
            c.n_ff = (int) num(ml, "expert", "ff", 0);
            c.n_expert = (int) num(ml, "router", "experts", 0);
            c.n_top = (int) num(ml, "router", "top", 0);
            c.moe_scale = (float) num(ml, "router", "scale", 1.0);
            if (const json_value * gr = ml->path("router", "groups")) {
                c.moe_groups = (int) num(gr, "count", nullptr, 1);
                c.moe_keep = (int) num(gr, "keep", nullptr, c.moe_groups);
            }
            if (c.n_ff <= 0 || c.n_expert <= 0 || c.n_top <= 0 || c.n_top > c.n_expert || c.moe_groups < 1 || c.moe_groups > 256 || c.n_expert % c.moe_groups || c.moe_keep < 1 ||
                c.moe_keep > c.moe_groups || c.n_top > c.moe_keep * (c.n_expert / c.moe_groups)) { err = lname + ": inconsistent router"; return false; }
        }
    }
    hp.n_head = m->lcfg[0].n_head; hp.n_head_kv = m->lcfg[0].n_head_kv; hp.n_embd_head = m->lcfg[0].dk; hp.n_ff = m->lcfg[0].n_ff;
    hp.rope_freq_base = m->lcfg[0].rot_base;
    for (int il = 0; il < (m->loop_times > 0 ? m->loop_start : hp.n_layer); ++il) m->runs.push_back({il, -1, false});
    if (m->loop_times > 0) {
        for (int t = 0; t < m->loop_times; ++t)
            for (int il = m->loop_start; il < m->loop_stop; ++il) m->runs.push_back({il, t, il == m->loop_start});
        for (int il = m->loop_stop; il < hp.n_layer; ++il) m->runs.push_back({il, -1, false});
    }
    return true;
}

static std::vector<dir_tensor> rarelorn_plan(const llm_model * m) {
    const llm_hparams & hp = m->hp;
    const ggml_type wt = m->wtype;
    const int64_t E = hp.n_embd;
    std::vector<dir_tensor> plan;
    auto add = [&](const std::string & name, ggml_type t, int64_t n0, int64_t n1, int64_t n2, std::vector<std::string> src, float gain) -> dir_tensor & {
        dir_tensor d;
        d.name = name; d.type = t; d.ne[0] = n0; d.ne[1] = n1; d.ne[2] = n2; d.src = std::move(src); d.synth_gain = gain;
        plan.push_back(std::move(d));
        return plan.back();
    };
    auto uniform = [&](dir_tensor & t, float lo, float hi) { t.synth_lo = lo; t.synth_hi = hi; };
    auto norm = [&](const std::string & name, const std::string & src) { uniform(add(name, GGML_TYPE_F32, E, 1, 1, {src}, 0.0f), 0.8f, 1.3f); plan.back().broadcast = true; };
    add("token_embd.weight", wt, E, hp.n_vocab, 1, {"embed"}, sqrtf((float) E));
    if (m->loop_times > 0) add("loop_step.weight", GGML_TYPE_F32, E, m->loop_times, 1, {"loop.step"}, sqrtf((float) E));
    for (int il = 0; il < hp.n_layer; ++il) {
        const llm_layer_cfg & c = m->lcfg[(size_t) il];
        const std::string p = "blk." + std::to_string(il) + ".", q = "l" + std::to_string(il) + ".", x = q + "mix.";
        const int64_t H = c.n_head, G = c.n_head_kv;
        norm(p + "attn_norm.weight", q + "norm1");
        if (c.mixer == LLM_MIX_MLSTM) {
            add(p + "attn_qkv.weight", wt, E, 2 * H * c.dk + H * c.dv, 1, {x + "q", x + "k", x + "v"}, 1.0f);
            add(p + "attn_gates.weight", wt, E, 2 * H, 1, {x + "i", x + "f"}, 2.0f);
            uniform(add(p + "attn_gates.bias", GGML_TYPE_F32, 2 * H, 1, 1, {x + "i.b", x + "f.b"}, 0.0f), -1.0f, 2.0f);
            add(p + "attn_gate.weight", wt, E, H * c.dv, 1, {x + "g"}, 1.0f);
            uniform(add(p + "attn_sub_norm.weight", GGML_TYPE_F32, H * c.dv, 1, 1, {x + "norm"}, 0.0f), 0.7f, 1.4f);
            add(p + "attn_output.weight", wt, H * c.dv, E, 1, {x + "o"}, 1.0f);
        } else if (c.mixer == LLM_MIX_DELTA) {
            const int64_t C = 2 * G * c.dk + H * c.dv;
            add(p + "attn_qkv.weight", wt, E, C, 1, {x + "q", x + "k", x + "v"}, 2.0f);
            add(p + "ssm_conv1d.weight", GGML_TYPE_F32, c.conv_taps, C, 1, {x + "q.conv", x + "k.conv", x + "v.conv"}, 1.0f);
            add(p + "attn_gates.weight", wt, E, 2 * H, 1, {x + "b", x + "a"}, 2.0f);
            uniform(add(p + "attn_gates.param", GGML_TYPE_F32, 2 * H, 1, 1, {x + "A_log", x + "dt_bias"}, 0.0f), -1.5f, 0.5f);
            add(p + "attn_gate.weight", wt, E, H * c.dv, 1, {x + "g"}, 1.0f);
            uniform(add(p + "attn_sub_norm.weight", GGML_TYPE_F32, c.dv, 1, 1, {x + "norm"}, 0.0f), 0.7f, 1.4f);
            add(p + "attn_output.weight", wt, H * c.dv, E, 1, {x + "o"}, 1.0f);
        } else {
            const std::string l = x + "left.", r = x + "right.";
            const int64_t C = H * c.dk + G * c.dk + G * c.dv, D = (int64_t) c.tm_heads * c.tm_dim;
            add(p + "attn_qkv.weight", wt, E, C, 1, {l + "q", l + "k", l + "v"}, 2.0f);
            add(p + "attn_qkv.bias", GGML_TYPE_F32, C, 1, 1, {l + "q.b", l + "k.b", l + "v.b"}, 0.3f * sqrtf((float) C));
            add(p + "ssm_conv1d.weight", GGML_TYPE_F32, c.conv_taps, C, 1, {l + "q.conv", l + "k.conv", l + "v.conv"}, 1.0f);
            uniform(add(p + "attn_fb.weight", GGML_TYPE_F32, H, 2, 1, {l + "temp", l + "pb"}, 0.0f), -2.0f, 1.5f);
            add(p + "attn_output.weight", wt, H * c.dv, E, 1, {l + "o"}, 1.0f);
            add(p + "attn_output.bias", GGML_TYPE_F32, E, 1, 1, {l + "o.b"}, 0.3f * sqrtf((float) E));
            add(p + "time_mix_taps.weight", GGML_TYPE_F32, 2, E, 5, {r + "mu.r", r + "mu.k", r + "mu.v", r + "mu.g", r + "mu.w"}, 0.0f).mix_taps = true;
            add(p + "time_mix_rkvg.weight", wt, E, D, 4, {r + "r", r + "k", r + "v", r + "g"}, 1.0f);
            add(p + "time_mix_w1.weight", wt, E, c.tm_rank, 1, {r + "w1"}, 1.0f);
            add(p + "time_mix_w2.weight", wt, c.tm_rank, D, 1, {r + "w2"}, 1.0f);
            uniform(add(p + "time_mix_w0.weight", GGML_TYPE_F32, D, 1, 1, {r + "w0"}, 0.0f), -3.0f, 0.0f);
            add(p + "time_mix_first.weight", GGML_TYPE_F32, c.tm_dim, c.tm_heads, 1, {r + "u"}, 0.5f * sqrtf((float) c.tm_dim));
            uniform(add(p + "time_mix_ln.weight", GGML_TYPE_F32, D, 1, 1, {r + "norm"}, 0.0f), 0.7f, 1.4f);
            add(p + "time_mix_output.weight", wt, D, E, 1, {r + "o"}, 1.0f);
        }
        if (c.mlp == LLM_MLP_MOE) {
            norm(p + "ffn_norm.weight", q + "norm2");
            std::vector<std::string> gu, downs;
            for (int e = 0; e < c.n_expert; ++e) {
                gu.push_back(q + "mlp.e" + std::to_string(e) + ".gate");
                gu.push_back(q + "mlp.e" + std::to_string(e) + ".up");
                downs.push_back(q + "mlp.e" + std::to_string(e) + ".down");
            }
            add(p + "ffn_gate_inp.weight", GGML_TYPE_F32, E, c.n_expert, 1, {q + "mlp.router"}, 3.0f);  // router logits are 32-bit in every mode
            add(p + "ffn_gate_up_exps.weight", wt, E, 2 * c.n_ff, c.n_expert, gu, 1.4f);                // per expert: its gate rows, then its up rows
            add(p + "ffn_down_exps.weight", wt, c.n_ff, E, c.n_expert, downs, 1.0f);
        }
    }
    norm("output_norm.weight", "final.norm");
    add("output.weight", wt, E, hp.n_vocab, 1, {"head"}, 1.0f);
    return plan;
}

// frequency of every rotation pair, base^(-2 i / dims), blended with its 1 / factor over the ramp between the two correction dims (YaRN); computed in f64
static std::vector<float> rope_frequencies(const llm_layer_cfg & c) {
    const int dims = c.rot_dims, half = dims / 2;
    std::vector<float> f((size_t) half);
    double lo = 0.0, hi = 0.0;
    if (c.yarn_factor > 0.0f) {
        auto corr = [&](double turns) { return dims * log((double) c.yarn_orig / (2.0 * M_PI * turns)) / (2.0 * log((double) c.rot_base)); };
        lo = std::max(floor(corr(c.yarn_fast)), 0.0);
        hi = std::min(ceil(corr(c.yarn_slow)), (double) dims - 1.0);
    }
    for (int i = 0; i < half; ++i) {
        const double fi = pow((double) c.rot_base, -2.0 * i / dims);
        double v = fi;
        if (c.yarn_factor > 0.0f) {
            const double ramp = std::min(1.0, std::max(0.0, (i - lo) / std::max(hi - lo, 0.001)));
            v = fi / c.yarn_factor * ramp + fi * (1.0 - ramp);
        }
        f[(size_t) i] = (float) v;
    }
    return f;
}
static float rope_magnitude(const llm_layer_cfg & c) { return c.yarn_factor > 0.0f ? (float) (0.1 * log((double) c.yarn_factor) + 1.0) : 1.0f; }

static std::vector<dir_tensor> zigipel_plan(const llm_model * m) {
    const llm_hparams & hp = m->hp;
    const ggml_type wt = m->wtype;
    const int64_t E = hp.n_embd;
    std::vector<dir_tensor> plan;
    auto add = [&](const std::string & name, ggml_type t, int64_t n0, int64_t n1, int64_t n2, std::vector<std::string> src, float gain) -> dir_tensor & {
        dir_tensor d;
        d.name = name; d.type = t; d.ne[0] = n0; d.ne[1] = n1; d.ne[2] = n2; d.src = std::move(src); d.synth_gain = gain;
        plan.push_back(std::move(d));
        return plan.back();
    };
    auto uniform = [&](dir_tensor & t, float lo, float hi) { t.synth_lo = lo; t.synth_hi = hi; };
    add("token_embd.weight", wt, E, hp.n_vocab, 1, {"embed"}, sqrtf((float) E));
    if (m->bg_buckets > 0) add("bigram_embd.weight", wt, E, m->bg_buckets + 1, 1, {"bigram"}, sqrtf((float) E));
    if (m->loop_times > 0) {
        add("loop_in.weight", wt, 2 * E, E, 1, {"loop.in"}, 1.4f);
        add("loop_step.weight", GGML_TYPE_F32, E, m->loop_times, 1, {"loop.step"}, 0.3f * sqrtf((float) E));
    }
    for (int il = 0; il < hp.n_layer; ++il) {
        const llm_layer_cfg & c = m->lcfg[(size_t) il];
        const std::string p = "blk." + std::to_string(il) + ".", q = "l" + std::to_string(il) + ".";
        const int64_t H = c.n_head;
        add(p + "attn_norm.weight", GGML_TYPE_F32, E, 1, 1, {q + "norm1"}, -1.0f);
        uniform(add(p + "shift.weight", GGML_TYPE_F32, E, 1, 1, {q + "shift"}, 0.0f), 0.0f, 1.0f);
        add(p + "attn_sink.weight", GGML_TYPE_F32, H, 1, 1, {q + "mix.sink"}, sqrtf((float) H));
        if (c.mixer == LLM_MIX_ATTN) {
            add(p + "attn_q.weight", wt, E, H * c.dk, 1, {q + "mix.q"}, 2.0f);
            add(p + "attn_k.weight", wt, E, (int64_t) c.n_head_kv * c.dk, 1, {q + "mix.k"}, 2.0f);
            add(p + "attn_v.weight", wt, E, (int64_t) c.n_head_kv * c.dv, 1, {q + "mix.v"}, 1.0f);
            add(p + "attn_gate.weight", wt, E, H, 1, {q + "mix.g"}, 1.0f);
            uniform(add(p + "attn_dist.weight", GGML_TYPE_F32, H, 1, 2, {q + "mix.r1", q + "mix.r2"}, 0.0f), 0.1f, 1.0f);  // r1 of every head, then r2 of every head
        } else {
            add(p + "attn_q.weight", wt, E, H * (c.dk + c.rot_dim), 1, {q + "mix.q"}, 2.0f);
            add(p + "attn_kv_a.weight", wt, E, c.kv_rank + c.rot_dim, 1, {q + "mix.dkv"}, 1.0f);
            add(p + "attn_kv_a_norm.weight", GGML_TYPE_F32, c.kv_rank, 1, 1, {q + "mix.dkv.norm"}, -1.0f);
            add(p + "attn_k_b_t.weight", wt, c.dk, c.kv_rank, H, {q + "mix.uk"}, 1.0f).head_transpose = true;
            add(p + "attn_v_b.weight", wt, c.kv_rank, c.dv, H, {q + "mix.uv"}, 1.0f);
            if (c.rot_dim > 0) add(p + "rope_freq.weight", GGML_TYPE_F32, c.rot_dim / 2, 1, 1, {}, 0.0f).values = rope_frequencies(c);
        }
        add(p + "attn_output.weight", wt, H * c.dv, E, 1, {q + "mix.o"}, 1.0f);
        if (c.mlp == LLM_MLP_DENSE) {
            add(p + "ffn_gate.weight", wt, E, c.n_ff, 1, {q + "mlp.gate"}, 1.0f);
            add(p + "ffn_gate.bias", GGML_TYPE_F32, c.n_ff, 1, 1, {q + "mlp.gate.b"}, 0.3f * sqrtf((float) c.n_ff));
            add(p + "ffn_up.weight", wt, E, c.n_ff, 1, {q + "mlp.up"}, 1.0f);
            add(p + "ffn_up.bias", GGML_TYPE_F32, c.n_ff, 1, 1, {q + "mlp.up.b"}, 0.3f * sqrtf((float) c.n_ff));
            add(p + "ffn_down.weight", wt, c.n_ff, E, 1, {q + "mlp.down"}, 1.0f);
            add(p + "ffn_down.bias", GGML_TYPE_F32, E, 1, 1, {q + "mlp.down.b"}, 0.3f * sqrtf((float) E));
        }
    }
    add("output_norm.weight", GGML_TYPE_F32, E, 1, 1, {"final.norm"}, -1.0f);
    add("output.weight", wt, E, hp.n_vocab, 1, {"head"}, 1.0f);
    return plan;
}

static std::vector<dir_tensor> nigozen_plan(const llm_model * m) {
    const llm_hparams & hp = m->hp;
    const ggml_type wt = m->wtype;
    const int64_t E = hp.n_embd;
    std::vector<dir_tensor> plan;
    auto add = [&](const std::string & name, ggml_type t, int64_t n0, int64_t n1, int64_t n2, std::vector<std::string> src, float gain) {
        dir_tensor d;
        d.name = name; d.type = t; d.ne[0] = n0; d.ne[1] = n1; d.ne[2] = n2; d.src = std::move(src); d.synth_gain = gain;
        plan.push_back(std::move(d));
    };
    add("token_embd.weight", wt, E, hp.n_vocab, 1, {"embed"}, sqrtf((float) E));
    int max_head = 1;
    for (int il = 0; il < hp.n_layer; ++il) {
        const llm_layer_cfg & c = m->lcfg[(size_t) il];
        const std::string p = "blk." + std::to_string(il) + ".", q = "l" + std::to_string(il) + ".";
        max_head = std::max(max_head, c.n_head);
        add(p + "attn_norm.weight", GGML_TYPE_F32, E, 1, 1, {q + "norm1"}, -1.0f);
        add(p + "attn_post_norm.weight", GGML_TYPE_F32, E, 1, 1, {q + "norm1b"}, -1.0f);
        add(p + "attn_q.weight", wt, E, (int64_t) c.n_head * c.dk, 1, {q + "mix.q"}, 2.0f);
        add(p + "attn_k.weight", wt, E, (int64_t) c.n_head_kv * c.dk, 1, {q + "mix.k"}, 2.0f);
        add(p + "attn_v.weight", wt, E, (int64_t) c.n_head_kv * c.dv, 1, {q + "mix.v"}, 1.0f);
        add(p + "attn_gate.weight", wt, E, (int64_t) c.n_head * c.dv, 1, {q + "mix.g"}, 1.0f);
        add(p + "attn_output.weight", wt, (int64_t) c.n_head * c.dv, E, 1, {q + "mix.o"}, 1.0f);
        if (c.mlp != LLM_MLP_NONE) {
            add(p + "ffn_norm.weight", GGML_TYPE_F32, E, 1, 1, {q + "norm2"}, -1.0f);
            add(p + "ffn_post_norm.weight", GGML_TYPE_F32, E, 1, 1, {q + "norm2b"}, -1.0f);
        }
        if (c.mlp == LLM_MLP_DENSE) {
            add(p + "ffn_up.weight", wt, E, c.n_ff, 1, {q + "mlp.up"}, 1.0f);
            add(p + "ffn_down.weight", wt, c.n_ff, E, 1, {q + "mlp.down"}, 1.0f);
        } else if (c.mlp == LLM_MLP_MOE) {
            std::vector<std::string> ups, downs;
            for (int e = 0; e < c.n_expert; ++e) {
                ups.push_back(q + "mlp.e" + std::to_string(e) + ".up");
                downs.push_back(q + "mlp.e" + std::to_string(e) + ".down");
            }
            add(p + "ffn_gate_inp.weight", GGML_TYPE_F32, E, c.n_expert, 1, {q + "mlp.router"}, 3.0f);  // router logits are 32-bit in every mode
            add(p + "ffn_up_exps.weight", wt, E, c.n_ff, c.n_expert, ups, 2.0f);
            add(p + "ffn_down_exps.weight", wt, c.n_ff, E, c.n_expert, downs, 1.0f);
        }
    }
    add("output_norm.weight", GGML_TYPE_F32, E, 1, 1, {"final.norm"}, -1.0f);
    add("attn_sinks.weight", GGML_TYPE_F32, max_head, 1, 1, {}, 0.0f);
    return plan;
}

// Nogavik: every layer is x += mixer(norm1(x)) + ff(norm2(x)) — two RMS norms of the same x whose weights are stored around zero (the loader adds 1) — followed by a
// per-layer token input: the layer's part e of a second embedding table, y = W_proj (gelu_tanh(W_gate x) * e), x += rms_norm(y) * w.  Mixers: latent attention whose
// queries come through a normed latent as well, neighbouring rotation pairs, a sigmoid output gate per value entry, and optionally the cache rows of an earlier layer
// instead of a down projection of its own (kv_from); a state-space mixer (Mamba-2); grouped-query attention with biases and per-head normed queries and keys (no
// rotation) beside a gated delta rule with one decay per key channel, the two outputs RMS-normed over the width and averaged.  Dense feed-forward with squared ReLU.
// The output matrix is the embedding table.
static bool parse_nogavik_config(const json_value & cfg, const st_file * file, llm_model * m, std::string & err) {
    llm_hparams & hp = m->hp;
    snprintf(hp.arch, sizeof(hp.arch), "nogavik");
    const json_value * layers = cfg.get("layers");
    if (!layers || layers->kind != json_value::ARR || layers->arr.empty()) { err = "config: no layers"; return false; }
    const json_value * v;
    hp.n_embd = (v = cfg.get("width")) ? (int) v->number(0) : 0;
    hp.n_vocab = (v = cfg.get("vocab")) ? (int) v->number(0) : 0;
    hp.rms_eps = (v = cfg.path("norm", "eps")) ? (float) v->number(1e-5) : 1e-5f;
    hp.n_layer = (int) layers->arr.size();
    hp.n_ctx_train = 1 << 20;
    if (hp.n_embd <= 0 || hp.n_vocab <= 0) { err = "config: width / vocab missing"; return false; }
    auto num = [&](const json_value * o, const char * k0, const char * k1, double d) { const json_value * x = o->path(k0, k1); return x ? x->number(d) : d; };
    const int side_dim = (v = cfg.path("token_side", "dim")) ? (int) v->number(0) : 0;
    if (side_dim < 0) { err = "config: inconsistent token_side"; return false; }
    m->lcfg.resize((size_t) hp.n_layer);
    m->has_attn = false;
    m->has_seq_state = false;
    m->hist_rows = 0;
    for (int il = 0; il < hp.n_layer; ++il) {
        const json_value & L = layers->arr[(size_t) il];
        llm_layer_cfg & c = m->lcfg[(size_t) il];
        const std::string lname = "config: layer " + std::to_string(il);
        const json_value * type = L.get("type");
        const json_value * mx = L.get("mixer");
        if (!type || type->kind != json_value::STR || !mx || mx->kind != json_value::OBJ) { err = lname + ": no mixer"; return false; }
        c.rms = c.parallel = c.two_norms = true;
        c.side_dim = side_dim;
        c.rot_dims = 0;
        if (type->str == "latent_attention") {
            c.mixer = LLM_MIX_LATENT;
            c.n_head = (int) num(mx, "heads", nullptr, 0);
            c.n_head_kv = 1;
            c.dk = (int) num(mx, "dim", nullptr, 0);
            c.dv = (int) num(mx, "vdim", nullptr, c.dk);
            c.kv_rank = (int) num(mx, "kv_rank", nullptr, 0);
            c.q_rank = (int) num(mx, "q_rank", nullptr, 0);
            c.rot_dim = (int) num(mx, "rot_dim", nullptr, 0);
            c.rot_dims = c.rot_dim;  // the rotated vector is the rot_dim part of a head, all of it
            c.rot_half = false;      // pairs are neighbours (2i, 2i + 1)
            c.rot_base = (float) num(mx, "rot", "base", 10000.0);
            c.scale = (float) num(mx, "scale", nullptr, c.dk + c.rot_dim > 0 ? 1.0 / sqrt((double) (c.dk + c.rot_dim)) : 1.0);
            c.out_gate = true;
            if (const json_value * kf = mx->path("kv_from")) c.kv_from = (int) kf->number(-1);
            if (c.n_head <= 0 || c.dk <= 0 || c.dv <= 0 || c.kv_rank <= 0 || c.q_rank <= 0 || c.rot_dim < 0 || (c.rot_dim & 1)) { err = lname + ": inconsistent latent attention sizes"; return false; }
            if (num(mx, "rot", "dims", c.rot_dim) != c.rot_dim) { err = lname + ": rot.dims differs from rot_dim"; return false; }
            if (mx->get("kv_from") && mx->get("kv_from")->kind != json_value::NUL) {
                const llm_layer_cfg * o = c.kv_from >= 0 && c.kv_from < il ? &m->lcfg[(size_t) c.kv_from] : nullptr;
                if (!o || o->mixer != LLM_MIX_LATENT || o->kv_from >= 0 || o->kv_rank != c.kv_rank || o->rot_dim != c.rot_dim || o->rot_base != c.rot_base) {
                    err = lname + ": kv_from names no earlier latent-attention layer with a down projection of its own and the same latent, rotated part and rotation";
                    return false;
                }
            }
            m->has_attn = true;
            m->max_embd_k = std::max(m->max_embd_k, c.kv_rank + c.rot_dim);
        } else if (type->str == "mamba2") {
            c.mixer = LLM_MIX_SSD;
            c.n_head = (int) num(mx, "heads", nullptr, 0);
            c.dv = (int) num(mx, "vdim", nullptr, 0);
            c.ssm_state = c.dk = (int) num(mx, "state", nullptr, 0);
            c.ssm_groups = c.n_head_kv = (int) num(mx, "groups", nullptr, 1);
            c.ssm_norm_groups = (int) num(mx, "norm_groups", nullptr, 1);
            c.conv_taps = (int) num(mx, "conv", nullptr, 1);
            if (c.n_head <= 0 || c.dv <= 0 || c.ssm_state <= 0 || c.ssm_state > 256 || c.ssm_groups <= 0 || c.n_head % c.ssm_groups || c.ssm_norm_groups <= 0 ||
                (c.n_head * c.dv) % c.ssm_norm_groups || c.conv_taps < 1 || c.conv_taps > 16) { err = lname + ": inconsistent state-space sizes"; return false; }
            m->has_seq_state = true;
        } else if (type->str == "parallel") {
            c.mixer = LLM_MIX_ATTN_DELTA;
            const json_value * lf = mx->get("left"), * rt = mx->get("right");
            if (!lf || lf->kind != json_value::OBJ || !rt || rt->kind != json_value::OBJ) { err = lname + ": a parallel mixer needs left and right"; return false; }
            c.n_head = (int) num(lf, "heads", nullptr, 0);
            c.n_head_kv = (int) num(lf, "kv_heads", nullptr, c.n_head);
            c.dk = (int) num(lf, "dim", nullptr, 0);
            c.dv = (int) num(lf, "vdim", nullptr, c.dk);
            c.scale = (float) num(lf, "scale", nullptr, c.dk > 0 ? 1.0 / sqrt((double) c.dk) : 1.0);
            c.qkv_bias = c.qk_norm = true;
            c.left_scale = c.right_scale = 0.5f;
            c.r_head = (int) num(rt, "heads", nullptr, 0);
            c.r_head_kv = (int) num(rt, "kv_heads", nullptr, c.r_head);
            c.r_dk = (int) num(rt, "dim", nullptr, 0);
            c.r_dv = (int) num(rt, "vdim", nullptr, c.r_dk);
            c.conv_taps = (int) num(rt, "conv", nullptr, 1);
            c.r_rank = (int) num(rt, "rank", nullptr, 16);  // (a checkpoint's a1 gives it)
            if (file) {
                const st_tensor * a1 = file->find("l" + std::to_string(il) + ".mix.right.a1");
                if (!a1 || a1->shape.size() != 2) { err = lname + ": no right.a1 in the checkpoint"; return false; }
                c.r_rank = (int) a1->shape[0];
            }
            if (c.n_head <= 0 || c.n_head_kv <= 0 || c.n_head % c.n_head_kv || c.dk <= 0 || c.dv <= 0 || c.r_head <= 0 || c.r_head_kv <= 0 || c.r_head % c.r_head_kv || c.r_dk <= 0 ||
                c.r_dk > 256 || c.r_dv <= 0 || c.r_rank <= 0 || c.conv_taps < 1 || c.conv_taps > 16) { err = lname + ": inconsistent parallel-mixer sizes"; return false; }
            m->has_attn = true;
            m->has_seq_state = true;
            m->max_embd_k = std::max(m->max_embd_k, c.n_head_kv * c.dk);
            m->max_embd_v = std::max(m->max_embd_v, c.n_head_kv * c.dv);
        } else { err = lname + ": unknown mixer type"; return false; }
        m->hist_rows = std::max(m->hist_rows, c.conv_taps - 1);
        c.mask_id = mask_rule_id(m, llm_mask_rule());  // every attention of the design is plainly causal
        const json_value * ml = L.path("mlp");
        if (ml && ml->kind == json_value::OBJ) {
            const json_value * kind = ml->get("kind");
            if (!kind || kind->kind != json_value::STR || kind->str != "dense") { err = lname + ": unknown mlp kind"; return false; }
            c.mlp = LLM_MLP_DENSE;
            c.ffn_relu_sq = true;
            c.n_ff = (int) num(ml, "ff", nullptr, 0);
            if (c.n_ff <= 0) { err = lname + ": ff missing"; return false; }
        }
    }
    hp.n_head = m->lcfg[0].n_head; hp.n_head_kv = m->lcfg[0].n_head_kv; hp.n_embd_head = m->lcfg[0].dk; hp.n_ff = m->lcfg[0].n_ff;
    hp.rope_freq_base = m->lcfg[0].rot_base;
    for (int il = 0; il < hp.n_layer; ++il) m->runs.push_back({il, -1, false});
    return true;
}

static std::vector<dir_tensor> nogavik_plan(const llm_model * m) {
    const llm_hparams & hp = m->hp;
    const ggml_type wt = m->wtype;
    const int64_t E = hp.n_embd;
    std::vector<dir_tensor> plan;
    auto add = [&](const std::string & name, ggml_type t, int64_t n0, int64_t n1, int64_t n2, std::vector<std::string> src, float gain) -> dir_tensor & {
        dir_tensor d;
        d.name = name; d.type = t; d.ne[0] = n0; d.ne[1] = n1; d.ne[2] = n2; d.src = std::move(src); d.synth_gain = gain;
        plan.push_back(std::move(d));
        return plan.back();
    };
    auto uniform = [&](dir_tensor & t, float lo, float hi) -> dir_tensor & { t.synth_lo = lo; t.synth_hi = hi; return t; };
    auto norm1p = [&](const std::string & name, const std::string & src) { uniform(add(name, GGML_TYPE_F32, E, 1, 1, {src}, 0.0f), -0.2f, 0.3f).one_plus = true; };  // 1 + w
    auto normw = [&](const std::string & name, int64_t n, const std::string & src) { uniform(add(name, GGML_TYPE_F32, n, 1, 1, {src}, 0.0f), 0.7f, 1.4f); };           // plain weight
    add("token_embd.weight", wt, E, hp.n_vocab, 1, {"embed"}, sqrtf((float) E));
    for (int il = 0; il < hp.n_layer; ++il) {
        const llm_layer_cfg & c = m->lcfg[(size_t) il];
        const std::string p = "blk." + std::to_string(il) + ".", q = "l" + std::to_string(il) + ".", x = q + "mix.";
        const int64_t H = c.n_head, G = c.n_head_kv;
        norm1p(p + "attn_norm.weight", q + "norm1");
        if (c.mixer == LLM_MIX_LATENT) {
            add(p + "attn_q_a.weight", wt, E, c.q_rank, 1, {x + "dq"}, 1.0f);
            normw(p + "attn_q_a_norm.weight", c.q_rank, x + "dq.norm");
            add(p + "attn_q.weight", wt, c.q_rank, H * (c.dk + c.rot_dim), 1, {x + "uq"}, 2.0f);
            if (c.kv_from < 0) {
                add(p + "attn_kv_a.weight", wt, E, c.kv_rank + c.rot_dim, 1, {x + "dkv"}, 1.0f);
                normw(p + "attn_kv_a_norm.weight", c.kv_rank, x + "dkv.norm");
            }
            add(p + "attn_k_b_t.weight", wt, c.dk, c.kv_rank, H, {x + "uk"}, 1.0f).head_transpose = true;
            add(p + "attn_v_b.weight", wt, c.kv_rank, c.dv, H, {x + "uv"}, 1.0f);
            if (c.rot_dim > 0) add(p + "rope_freq.weight", GGML_TYPE_F32, c.rot_dim / 2, 1, 1, {}, 0.0f).values = rope_frequencies(c);
            add(p + "attn_gate.weight", wt, E, H * c.dv, 1, {x + "g"}, 1.0f);
            add(p + "attn_output.weight", wt, H * c.dv, E, 1, {x + "o"}, 1.0f);
        } else if (c.mixer == LLM_MIX_SSD) {
            const int64_t inner = H * c.dv, GN = (int64_t) c.ssm_groups * c.ssm_state, ch = inner + 2 * GN;
            // the input projection [z | x, B, C | dt] is kept in its three parts: each is read whole by what follows it
            add(p + "ssm_in_z.weight", wt, E, inner, 1, {x + "in"}, 1.0f).row0 = 0;
            add(p + "ssm_in_xbc.weight", wt, E, ch, 1, {x + "in"}, 2.0f).row0 = inner;
            add(p + "ssm_in_dt.weight", wt, E, H, 1, {x + "in"}, 2.0f).row0 = inner + ch;
            add(p + "ssm_conv1d.weight", GGML_TYPE_F32, c.conv_taps, ch, 1, {x + "conv"}, 1.0f);
            add(p + "ssm_conv1d.bias", GGML_TYPE_F32, ch, 1, 1, {x + "conv.b"}, 0.3f * sqrtf((float) ch));
            uniform(add(p + "ssm_params.weight", GGML_TYPE_F32, 3 * H, 1, 1, {x + "A_log", x + "dt_bias", x + "D"}, 0.0f), -1.5f, 0.5f);
            normw(p + "attn_sub_norm.weight", inner, x + "norm");
            add(p + "attn_output.weight", wt, inner, E, 1, {x + "o"}, 1.0f);
        } else {
            const std::string l = x + "left.", r = x + "right.";
            add(p + "attn_q.weight", wt, E, H * c.dk, 1, {l + "q"}, 2.0f);
            add(p + "attn_k.weight", wt, E, G * c.dk, 1, {l + "k"}, 2.0f);
            add(p + "attn_v.weight", wt, E, G * c.dv, 1, {l + "v"}, 1.0f);
            add(p + "attn_q.bias", GGML_TYPE_F32, H * c.dk, 1, 1, {l + "q.b"}, 0.3f * sqrtf((float) (H * c.dk)));
            add(p + "attn_k.bias", GGML_TYPE_F32, G * c.dk, 1, 1, {l + "k.b"}, 0.3f * sqrtf((float) (G * c.dk)));
            add(p + "attn_v.bias", GGML_TYPE_F32, G * c.dv, 1, 1, {l + "v.b"}, 0.3f * sqrtf((float) (G * c.dv)));
            normw(p + "attn_q_norm.weight", c.dk, l + "q.norm");
            normw(p + "attn_k_norm.weight", c.dk, l + "k.norm");
            add(p + "attn_output.weight", wt, H * c.dv, E, 1, {l + "o"}, 1.0f);
            normw(p + "mix_left_norm.weight", E, l + "out");
            const int64_t RH = c.r_head, RG = c.r_head_kv, C = 2 * RG * c.r_dk + RH * c.r_dv;
            add(p + "attn_qkv.weight", wt, E, C, 1, {r + "q", r + "k", r + "v"}, 2.0f);
            add(p + "ssm_conv1d.weight", GGML_TYPE_F32, c.conv_taps, C, 1, {r + "q.conv", r + "k.conv", r + "v.conv"}, 1.0f);
            add(p + "delta_beta.weight", wt, E, RH, 1, {r + "b"}, 2.0f);
            add(p + "delta_a1.weight", wt, E, c.r_rank, 1, {r + "a1"}, 1.0f);
            add(p + "delta_a2.weight", wt, c.r_rank, RH * c.r_dk, 1, {r + "a2"}, 2.0f);
            uniform(add(p + "attn_gates.param", GGML_TYPE_F32, RH + RH * c.r_dk, 1, 1, {r + "A_log", r + "dt_bias"}, 0.0f), -1.5f, 0.5f);
            add(p + "delta_g1.weight", wt, E, c.r_rank, 1, {r + "g1"}, 1.0f);
            add(p + "delta_g2.weight", wt, c.r_rank, RH * c.r_dv, 1, {r + "g2"}, 2.0f);
            normw(p + "attn_sub_norm.weight", c.r_dv, r + "norm");
            add(p + "delta_output.weight", wt, RH * c.r_dv, E, 1, {r + "o"}, 1.0f);
            normw(p + "mix_right_norm.weight", E, r + "out");
        }
        if (c.mlp == LLM_MLP_DENSE) {
            norm1p(p + "ffn_norm.weight", q + "norm2");
            add(p + "ffn_up.weight", wt, E, c.n_ff, 1, {q + "mlp.up"}, 1.4f);
            add(p + "ffn_down.weight", wt, c.n_ff, E, 1, {q + "mlp.down"}, 1.0f);
        }
        if (c.side_dim > 0) {
            add(p + "side_embd.weight", wt, c.side_dim, hp.n_vocab, 1, {"side.embed"}, sqrtf((float) c.side_dim)).col0 = (int64_t) il * c.side_dim;
            add(p + "side_gate.weight", wt, E, c.side_dim, 1, {q + "side.gate"}, 1.0f);
            add(p + "side_proj.weight", wt, c.side_dim, E, 1, {q + "side.proj"}, 1.0f);
            normw(p + "side_norm.weight", E, q + "side.norm");
        }
    }
    norm1p("output_norm.weight", "final.norm");
    return plan;
}

// values of one checkpoint tensor (bf16 / f32 / f16 in the file) as `type` (bf16 or f32) into dst
static bool convert_values(const st_tensor & t, ggml_type type, uint8_t * dst) {
    const int64_t n = t.numel();
    for (int64_t i = 0; i < n; ++i) {
        float f;
        if (t.dtype == "BF16") { uint16_t h; memcpy(&h, t.data + i * 2, 2); if (type == GGML_TYPE_BF16) { memcpy(dst + i * 2, &h, 2); continue; } f = bf16_to_f32(h); }
        else if (t.dtype == "F32") memcpy(&f, t.data + i * 4, 4);
        else if (t.dtype == "F16") { uint16_t h; memcpy(&h, t.data + i * 2, 2); f = f16_to_f32(h); }
        else return false;
        if (type == GGML_TYPE_F32) memcpy(dst + i * 4, &f, 4);
        else { const uint16_t h = f32_to_bf16(f); memcpy(dst + i * 2, &h, 2); }
    }
    return true;
}

static float gauss(uint64_t & s) {  // Box-Muller on two uniforms
    const float u1 = std::max(u01(splitmix64(s)), 1e-7f), u2 = u01(splitmix64(s));
    return sqrtf(-2.0f * logf(u1)) * cosf(6.2831853f * u2);
}

static llm_model * model_from_config(const json_value & cfg, const st_file * file, uint64_t seed, ggml_backend_buffer_type_t buft, int wtype) {
    const json_value * arch = cfg.get("architecture");
    if (!arch || arch->kind != json_value::STR) { fprintf(stderr, "llm_model_load_dir: config.json names no architecture\n"); return nullptr; }
    if (wtype != GGML_TYPE_BF16 && wtype != GGML_TYPE_F32) { fprintf(stderr, "llm_model_load_dir: matrices are kept as bf16 or f32\n"); return nullptr; }
    llm_model * m = new llm_model();
    m->wtype = (ggml_type) wtype;
    std::string err;
    // the registry of model classes that are described by a config.json
    std::vector<dir_tensor> plan;
    if (arch->str == "Nigozen") {
        if (!parse_nigozen_config(cfg, m, err)) { fprintf(stderr, "llm_model_load_dir: %s\n", err.c_str()); delete m; return nullptr; }
        plan = nigozen_plan(m);
    } else if (arch->str == "Zigipel") {
        if (!parse_zigipel_config(cfg, m, err)) { fprintf(stderr, "llm_model_load_dir: %s\n", err.c_str()); delete m; return nullptr; }
        plan = zigipel_plan(m);
    } else if (arch->str == "Rarelorn") {
        if (!parse_rarelorn_config(cfg, file, m, err)) { fprintf(stderr, "llm_model_load_dir: %s\n", err.c_str()); delete m; return nullptr; }
        plan = rarelorn_plan(m);
    } else if (arch->str == "Nogavik") {
        if (!parse_nogavik_config(cfg, file, m, err)) { fprintf(stderr, "llm_model_load_dir: %s\n", err.c_str()); delete m; return nullptr; }
        plan = nogavik_plan(m);
    } else {
        fprintf(stderr, "llm_model_load_dir: unknown architecture \"%s\"\n", arch->str.c_str());
        delete m;
        return nullptr;
    }
    m->ctx = ggml_init({0, nullptr, true});
    for (auto & t : plan) {
        // shapes are checked against the file before anything is allocated
        if (file && (t.row0 >= 0 || t.col0 >= 0)) {
            // a part of ONE stored matrix: some of its rows, or some columns of every row
            const st_tensor * st = t.src.size() == 1 ? file->find(t.src[0]) : nullptr;
            const bool ok = st && st->shape.size() == 2 && t.ne[2] == 1 &&
                            (t.row0 >= 0 ? st->shape[1] == t.ne[0] && t.row0 + t.ne[1] <= st->shape[0] : st->shape[0] == t.ne[1] && t.col0 + t.ne[0] <= st->shape[1]);
            if (!ok) {
                fprintf(stderr, "llm_model_load_dir: tensor %s (a part of %s) is missing or has another shape than the config implies\n", t.name.c_str(), t.src.empty() ? "?" : t.src[0].c_str());
                llm_model_free(m);
                return nullptr;
            }
        } else if (file && (t.broadcast || t.mix_taps || (t.src.size() > 1 && t.ne[2] == 1))) {
            // one number for a whole row; shift factors of ne1 entries each; or matrices / vectors of UNEQUAL heights stacked along dim 1 (q, k, v as one projection)
            int64_t total = 0;
            bool ok = true;
            for (auto & sname : t.src) {
                const st_tensor * st = file->find(sname);
                if (!st) { ok = false; break; }
                total += st->numel();
                if (t.broadcast) ok = ok && st->numel() == 1;
                else if (t.mix_taps) ok = ok && st->numel() == t.ne[1];
                else ok = ok && (st->shape.size() == 2 ? st->shape[1] == t.ne[0] : (st->shape.size() == 1 && (t.ne[0] == 1 || t.ne[1] == 1 || st->shape[0] == t.ne[0])));
            }
            if (!t.broadcast && !t.mix_taps) ok = ok && total == t.ne[0] * t.ne[1];
            if (!ok) {
                fprintf(stderr, "llm_model_load_dir: tensor %s (from %s ...) is missing or has another shape than the config implies\n", t.name.c_str(), t.src[0].c_str());
                llm_model_free(m);
                return nullptr;
            }
        } else if (file)
            for (auto & sname : t.src) {
                const st_tensor * st = file->find(sname);
                const int64_t n_src = (int64_t) t.src.size(), want = t.ne[0] * t.ne[1] * t.ne[2] / n_src;
                const int64_t cols = t.head_transpose ? t.ne[1] : t.ne[0], rows = t.head_transpose ? t.ne[0] * t.ne[2] : t.ne[1] * t.ne[2] / n_src;
                if (!st || st->numel() != want || (st->shape.size() == 2 && (st->shape[1] != cols || st->shape[0] != rows))) {
                    fprintf(stderr, "llm_model_load_dir: tensor %s is missing or has another shape than the config implies\n", sname.c_str());
                    llm_model_free(m);
                    return nullptr;
                }
            }
        ggml_tensor * x = ggml_new_tensor_3d(m->ctx, t.type, t.ne[0], t.ne[1], t.ne[2]);
        ggml_set_name(x, t.name.c_str());
    }
    ggml_backend_buffer_t buf = ggml_backend_alloc_ctx_tensors_from_buft(m->ctx, buft);
    if (!buf) { fprintf(stderr, "llm_model_load_dir: failed to allocate weights\n"); llm_model_free(m); return nullptr; }
    ggml_backend_buffer_set_usage(buf, GGML_BACKEND_BUFFER_USAGE_WEIGHTS);
    m->buffers.push_back(buf);
    std::vector<uint8_t> stage;
    int tid = 0;
    for (auto & t : plan) {
        ggml_tensor * x = ggml_get_tensor(m->ctx, t.name.c_str());
        const size_t esz = ggml_type_size(t.type), total = (size_t) (t.ne[0] * t.ne[1] * t.ne[2]) * esz, slice = t.src.empty() ? total : total / t.src.size();
        stage.assign(total, 0);
        ++tid;
        if (!t.values.empty()) {
            LLM_ASSERT(t.type == GGML_TYPE_F32 && t.values.size() * 4 == total);
            memcpy(stage.data(), t.values.data(), total);
        } else if (t.src.empty()) {
            // zeros (the sinks)
        } else if (file && (t.row0 >= 0 || t.col0 >= 0)) {
            const st_tensor * st = file->find(t.src[0]);
            std::vector<uint8_t> whole((size_t) st->numel() * esz);
            if (!convert_values(*st, t.type, whole.data())) { fprintf(stderr, "llm_model_load_dir: tensor %s has an unsupported dtype\n", t.src[0].c_str()); llm_model_free(m); return nullptr; }
            if (t.row0 >= 0) memcpy(stage.data(), whole.data() + (size_t) (t.row0 * t.ne[0]) * esz, total);
            else for (int64_t r = 0; r < t.ne[1]; ++r) memcpy(stage.data() + (size_t) (r * t.ne[0]) * esz, whole.data() + (size_t) (r * st->shape[1] + t.col0) * esz, (size_t) t.ne[0] * esz);
        } else if (file && (t.broadcast || t.mix_taps)) {
            LLM_ASSERT(t.type == GGML_TYPE_F32);
            float * out = (float *) stage.data();
            std::vector<uint8_t> tmp;
            for (size_t k = 0; k < t.src.size(); ++k) {
                const st_tensor * st = file->find(t.src[k]);
                tmp.resize((size_t) st->numel() * 4);
                if (!convert_values(*st, GGML_TYPE_F32, tmp.data())) { fprintf(stderr, "llm_model_load_dir: tensor %s has an unsupported dtype\n", t.src[k].c_str()); llm_model_free(m); return nullptr; }
                const float * in = (const float *) tmp.data();
                if (t.broadcast) for (int64_t i = 0; i < t.ne[0] * t.ne[1] * t.ne[2]; ++i) out[i] = in[0];
                else for (int64_t i = 0; i < t.ne[1]; ++i) { out[(k * t.ne[1] + i) * 2] = in[i]; out[(k * t.ne[1] + i) * 2 + 1] = 1.0f - in[i]; }
            }
        } else if (file) {
            size_t at = 0;  // (sources of unequal sizes follow one another)
            for (size_t k = 0; k < t.src.size(); ++k) {
                const st_tensor * stk = file->find(t.src[k]);
                const size_t off = at;
                at += (size_t) stk->numel() * esz;
                LLM_ASSERT(at <= total);
                (void) slice;
                if (!convert_values(*stk, t.type, stage.data() + off)) {
                    fprintf(stderr, "llm_model_load_dir: tensor %s has an unsupported dtype\n", t.src[k].c_str());
                    llm_model_free(m);
                    return nullptr;
                }
            }
            if (t.head_transpose) {  // file: [head][row r][col c]  ->  kept: [head][col c][row r] (rows along dim 0)
                std::vector<uint8_t> tr(total);
                const int64_t R = t.ne[0], Cc = t.ne[1];
                for (int64_t h = 0; h < t.ne[2]; ++h)
                    for (int64_t r = 0; r < R; ++r)
                        for (int64_t cc = 0; cc < Cc; ++cc)
                            memcpy(tr.data() + (size_t) ((h * Cc + cc) * R + r) * esz, stage.data() + (size_t) ((h * R + r) * Cc + cc) * esz, esz);
                stage.swap(tr);
            }
        } else if (t.mix_taps) {
            uint64_t s = seed ^ ((uint64_t) tid * 0xD1B54A32D192ED03ull);
            float * out = (float *) stage.data();
            for (int64_t i = 0; i < t.ne[1] * t.ne[2]; ++i) {
                const float mu = bf16_to_f32(f32_to_bf16(0.05f + 0.9f * u01(splitmix64(s))));
                out[2 * i] = mu;
                out[2 * i + 1] = 1.0f - mu;
            }
        } else if (t.synth_hi > t.synth_lo) {
            uint64_t s = seed ^ ((uint64_t) tid * 0xD1B54A32D192ED03ull);
            const int64_t n = t.ne[0] * t.ne[1] * t.ne[2];
            for (int64_t i = 0; i < n; ++i) {
                const float f = bf16_to_f32(f32_to_bf16(t.synth_lo + (t.synth_hi - t.synth_lo) * u01(splitmix64(s))));
                LLM_ASSERT(t.type == GGML_TYPE_F32);
                memcpy(stage.data() + i * 4, &f, 4);
            }
        } else {
            uint64_t s = seed ^ ((uint64_t) tid * 0xD1B54A32D192ED03ull);
            const int64_t n = t.ne[0] * t.ne[1] * t.ne[2];
            const float g = t.synth_gain / sqrtf((float) t.ne[0]);
            for (int64_t i = 0; i < n; ++i) {
                const float f = t.synth_gain < 0.0f ? 1.0f + 0.1f * gauss(s) : g * gauss(s);
                if (t.type == GGML_TYPE_F32) memcpy(stage.data() + i * 4, &f, 4);
                else { const uint16_t h = f32_to_bf16(f); memcpy(stage.data() + i * 2, &h, 2); }
            }
        }
        if (t.one_plus) {  // (the sum is rounded to f32 once, here)
            LLM_ASSERT(t.type == GGML_TYPE_F32);
            float * out = (float *) stage.data();
            for (int64_t i = 0; i < t.ne[0] * t.ne[1] * t.ne[2]; ++i) out[i] += 1.0f;
        }
        ggml_backend_tensor_set(x, stage.data(), 0, stage.size());
        m->total_bytes += stage.size();
    }
    // bind
    m->tok_embd = ggml_get_tensor(m->ctx, "token_embd.weight");
    m->output = ggml_get_tensor(m->ctx, "output.weight");
    if (!m->output) m->output = m->tok_embd;  // no output matrix of its own: the embedding table itself
    m->output_norm = ggml_get_tensor(m->ctx, "output_norm.weight");
    m->attn_sinks = ggml_get_tensor(m->ctx, "attn_sinks.weight");
    m->bigram = ggml_get_tensor(m->ctx, "bigram_embd.weight");
    m->loop_in = ggml_get_tensor(m->ctx, "loop_in.weight");
    m->loop_step = ggml_get_tensor(m->ctx, "loop_step.weight");
    m->layers.resize((size_t) m->hp.n_layer);
    uint64_t sbytes = ggml_nbytes(m->tok_embd) + ggml_nbytes(m->output_norm);
    if (m->output != m->tok_embd) sbytes = ggml_nbytes(m->output) + ggml_nbytes(m->output_norm) + ggml_row_size(m->tok_embd->type, m->hp.n_embd) * (m->bigram ? 2 : 1);
    std::vector<int> times_run((size_t) m->hp.n_layer, 0);
    for (const llm_run & r : m->runs) times_run[(size_t) r.il]++;
    if (m->loop_in) sbytes += (uint64_t) m->loop_times * (ggml_nbytes(m->loop_in) + ggml_row_size(GGML_TYPE_F32, m->hp.n_embd));
    for (int il = 0; il < m->hp.n_layer; ++il) {
        const std::string p = "blk." + std::to_string(il) + ".";
        auto g = [&](const char * s) { return ggml_get_tensor(m->ctx, (p + s).c_str()); };
        llm_layer & L = m->layers[(size_t) il];
        llm_layer_cfg & c = m->lcfg[(size_t) il];
        L.attn_norm = g("attn_norm.weight"); L.attn_post_norm = g("attn_post_norm.weight"); L.wq = g("attn_q.weight"); L.wk = g("attn_k.weight");
        L.wv = g("attn_v.weight"); L.attn_gate = g("attn_gate.weight"); L.wo = g("attn_output.weight");
        L.ffn_norm = g("ffn_norm.weight"); L.ffn_post_norm = g("ffn_post_norm.weight"); L.ffn_up = g("ffn_up.weight"); L.ffn_down = g("ffn_down.weight");
        L.ffn_gate_inp = g("ffn_gate_inp.weight"); L.ffn_up_exps = g("ffn_up_exps.weight"); L.ffn_down_exps = g("ffn_down_exps.weight");
        L.attn_sink = g("attn_sink.weight"); L.attn_r12 = g("attn_dist.weight"); L.shift = g("shift.weight");
        L.ffn_gate = g("ffn_gate.weight"); L.ffn_gate_b = g("ffn_gate.bias"); L.ffn_up_b = g("ffn_up.bias"); L.ffn_down_b = g("ffn_down.bias");
        L.wqkv = g("attn_qkv.weight"); L.bqkv = g("attn_qkv.bias"); L.conv = g("ssm_conv1d.weight"); L.wgates = g("attn_gates.weight");
        L.gate_par = g("attn_gates.bias") ? g("attn_gates.bias") : g("attn_gates.param"); L.sub_norm = g("attn_sub_norm.weight"); L.bo = g("attn_output.bias"); L.attn_fb = g("attn_fb.weight");
        L.tm_taps = g("time_mix_taps.weight"); L.tm_rkvg = g("time_mix_rkvg.weight"); L.tm_w1 = g("time_mix_w1.weight"); L.tm_w2 = g("time_mix_w2.weight"); L.tm_w0 = g("time_mix_w0.weight");
        L.tm_u = g("time_mix_first.weight"); L.tm_norm = g("time_mix_ln.weight"); L.tm_out = g("time_mix_output.weight"); L.ffn_gate_up_exps = g("ffn_gate_up_exps.weight");
        L.bq = g("attn_q.bias"); L.bk = g("attn_k.bias"); L.bv = g("attn_v.bias"); L.q_norm = g("attn_q_norm.weight"); L.k_norm = g("attn_k_norm.weight");
        L.wdq = g("attn_q_a.weight"); L.dq_norm = g("attn_q_a_norm.weight");
        L.wbeta = g("delta_beta.weight"); L.wa1 = g("delta_a1.weight"); L.wa2 = g("delta_a2.weight"); L.wg1 = g("delta_g1.weight"); L.wg2 = g("delta_g2.weight");
        L.wo_r = g("delta_output.weight"); L.left_norm = g("mix_left_norm.weight"); L.right_norm = g("mix_right_norm.weight");
        L.ssm_in_z = g("ssm_in_z.weight"); L.ssm_in_xbc = g("ssm_in_xbc.weight"); L.ssm_in_dt = g("ssm_in_dt.weight"); L.conv_b = g("ssm_conv1d.bias");
        if (!L.gate_par) L.gate_par = g("ssm_params.weight");
        L.side_embd = g("side_embd.weight"); L.side_gate = g("side_gate.weight"); L.side_proj = g("side_proj.weight"); L.side_norm = g("side_norm.weight");
        L.wdkv = g("attn_kv_a.weight"); L.dkv_norm = g("attn_kv_a_norm.weight"); L.wuk_t = g("attn_k_b_t.weight"); L.wuv = g("attn_v_b.weight"); L.rope_freq = g("rope_freq.weight");
        for (ggml_tensor * t : {L.attn_norm, L.attn_post_norm, L.wq, L.wk, L.wv, L.attn_gate, L.wo, L.ffn_norm, L.ffn_post_norm, L.ffn_up, L.ffn_down, L.ffn_gate_inp,
                                L.attn_sink, L.attn_r12, L.shift, L.ffn_gate, L.ffn_gate_b, L.ffn_up_b, L.ffn_down_b, L.wdkv, L.dkv_norm, L.wuk_t, L.wuv, L.rope_freq,
                                L.wqkv, L.bqkv, L.conv, L.wgates, L.gate_par, L.sub_norm, L.bo, L.attn_fb, L.tm_taps, L.tm_rkvg, L.tm_w1, L.tm_w2, L.tm_w0, L.tm_u, L.tm_norm, L.tm_out,
                                L.bq, L.bk, L.bv, L.q_norm, L.k_norm, L.wdq, L.dq_norm, L.wbeta, L.wa1, L.wa2, L.wg1, L.wg2, L.wo_r, L.left_norm, L.right_norm, L.ssm_in_z, L.ssm_in_xbc,
                                L.ssm_in_dt, L.conv_b, L.side_gate, L.side_proj, L.side_norm})
            if (t) sbytes += ggml_nbytes(t) * (uint64_t) std::max(1, times_run[(size_t) il]);  // (a layer of a repeated range is streamed once per run)
        if (L.side_embd) sbytes += ggml_row_size(L.side_embd->type, L.side_embd->ne[0]);  // (one row of the layer's part of the side table)
        if (c.mlp == LLM_MLP_MOE) sbytes += (ggml_nbytes(L.ffn_gate_up_exps ? L.ffn_gate_up_exps : L.ffn_up_exps) + ggml_nbytes(L.ffn_down_exps)) / (uint64_t) c.n_expert * (uint64_t) c.n_top *
                                            (uint64_t) std::max(1, times_run[(size_t) il]);
        if (c.v_mix) {  // the blend factor is a scalar of the checkpoint, read once
            float lam = 0.5f;
            if (file) {
                const st_tensor * st = file->find("l" + std::to_string(il) + ".mix.vmix");
                if (!st || st->numel() != 1) { fprintf(stderr, "llm_model_load_dir: layer %d has no scalar mix.vmix\n", il); llm_model_free(m); return nullptr; }
                uint8_t tmp[4];
                if (!convert_values(*st, GGML_TYPE_F32, tmp)) { llm_model_free(m); return nullptr; }
                memcpy(&lam, tmp, 4);
            } else {
                uint64_t s = seed ^ (0xABCDull + (uint64_t) il);
                lam = bf16_to_f32(f32_to_bf16(0.2f + 0.6f * u01(splitmix64(s))));
            }
            c.v_lambda = lam;
        }
    }
    m->stream_bytes = sbytes;
    m->n_head_l = m->hp.n_head; m->n_head_kv_l = m->hp.n_head_kv; m->n_ff_l = m->hp.n_ff;
    m->n_vocab_l = m->hp.n_vocab;
    return m;
}

extern "C" struct llm_model * llm_model_load_dir(const char * dir, ggml_backend_buffer_type_t buft, int wtype) {
    const std::string d = dir;
    std::string text;
    {
        FILE * f = fopen((d + "/config.json").c_str(), "rb");
        if (!f) { fprintf(stderr, "llm_model_load_dir: %s/config.json cannot be read\n", dir); return nullptr; }
        char buf[65536];
        size_t n;
        while ((n = fread(buf, 1, sizeof(buf), f)) > 0) text.append(buf, n);
        fclose(f);
    }
    json_value cfg;
    if (!json_parser::parse(text.data(), text.size(), cfg) || cfg.kind != json_value::OBJ) { fprintf(stderr, "llm_model_load_dir: %s/config.json is not a JSON object\n", dir); return nullptr; }
    st_file * file = st_file::open((d + "/model.safetensors").c_str());
    if (!file) return nullptr;
    llm_model * m = model_from_config(cfg, file, 0, buft, wtype);
    delete file;
    return m;
}
extern "C" struct llm_model * llm_model_synth_config(const char * config_json, uint64_t seed, ggml_backend_buffer_type_t buft, int wtype) {
    json_value cfg;
    if (!config_json || !json_parser::parse(config_json, strlen(config_json), cfg) || cfg.kind != json_value::OBJ) { fprintf(stderr, "llm_model_synth_config: the text is not a JSON object\n"); return nullptr; }
    return model_from_config(cfg, nullptr, seed, buft, wtype);
}

extern "C" void llm_model_free(struct llm_model * m) {
    if (!m) return;
    for (auto b : m->buffers) ggml_backend_buffer_free(b);
    ggml_free(m->ctx);
    delete m;
}
extern "C" const struct llm_hparams * llm_model_hparams(const struct llm_model * m) { return &m->hp; }
extern "C" uint64_t llm_model_stream_bytes(const struct llm_model * m) { return m->stream_bytes; }
extern "C" uint64_t llm_model_total_bytes(const struct llm_model * m) { return m->total_bytes; }
extern "C" struct ggml_tensor * llm_model_tensor(struct llm_model * m, const char * name) { return ggml_get_tensor(m->ctx, name); }

// ---------------------------------------------------------------------------------------------- context
// one row of the attention mask: `vis` where the cell holds a position of sequence s that is not after p, `hid` elsewhere (written to
// vectorise — no short-circuit — and compiled at -O3: the library is built at -O2, where this compiler does not try)
#pragma GCC push_options
#pragma GCC optimize("O3")
static void mask_row(float * __restrict__ row, const int n_kv, const int32_t * __restrict__ cpos, const int32_t * __restrict__ cseq, const int32_t s, const int32_t p,
                     const float vis, const float hid) {
    const uint32_t pu = (uint32_t) p;
    for (int j = 0; j < n_kv; ++j) {
        const bool v = (cseq[j] == s) & ((uint32_t) cpos[j] <= pu);
        row[j] = v ? vis : hid;
    }
}
// the same with attention confined to chunks of `chunk` positions counted from position 0 of the sequence: cell j is visible to position p only when
// floor(pos_j / chunk) == floor(p / chunk) as well (where a prompt was cut for processing plays no part: the rule reads positions only)
static void mask_row_chunked(float * __restrict__ row, const int n_kv, const int32_t * __restrict__ cpos, const int32_t * __restrict__ cseq, const int32_t s, const int32_t p,
                             const int32_t chunk, const float vis, const float hid) {
    const int32_t lo = p / chunk * chunk;  // first position of p's chunk
    const uint32_t span = (uint32_t) (p - lo);
    for (int j = 0; j < n_kv; ++j) {
        const bool v = (cseq[j] == s) & ((uint32_t) (cpos[j] - lo) <= span);  // lo <= pos_j <= p (an empty cell's -1 wraps to a huge value)
        row[j] = v ? vis : hid;
    }
}
// a sliding window that also keeps the first positions: cell j is visible to position p when pos_j <= p and (p - pos_j < window or pos_j < keep_first).
// A visible cell's entry is 0, or — `distance` — p - pos_j itself, for layers whose scores carry a penalty on the distance
static void mask_row_window(float * __restrict__ row, const int n_kv, const int32_t * __restrict__ cpos, const int32_t * __restrict__ cseq, const int32_t s, const int32_t p,
                            const int32_t window, const int32_t keep_first, const bool distance, const float hid) {
    const uint32_t pu = (uint32_t) p, wu = window > 0 ? (uint32_t) window : 0xFFFFFFFFu, ku = (uint32_t) keep_first;
    for (int j = 0; j < n_kv; ++j) {
        const uint32_t d = (uint32_t) (p - cpos[j]);  // (an empty cell's -1 gives p + 1: hidden by the first test)
        const bool v = (cseq[j] == s) & ((uint32_t) cpos[j] <= pu) & ((d < wu) | ((uint32_t) cpos[j] < ku));
        row[j] = v ? (distance ? (float) d : 0.0f) : hid;
    }
}
#pragma GCC pop_options

struct kv_cell {
    int32_t pos = -1;
    int32_t seq = -1;
};

// the inputs a graph segment reads and the tensor it ends in.  One segment = the whole model on one backend; with -sm layer one segment per device,
// each with its own copies of the inputs and, from the second on, the residual stream of the previous device as an input (`resid`)
struct seg_io {
    ggml_tensor *tokens = nullptr, *pos = nullptr, *mask = nullptr, *k_idxs = nullptr, *v_idxs = nullptr, *out_ids = nullptr, *resid = nullptr;
    ggml_tensor * out = nullptr;  // l_out of the segment's last layer, or the logits
    std::vector<ggml_tensor *> masks;  // models whose layers differ in what they may see: one mask per distinct rule (masks[0] == mask)
    ggml_tensor * bigram_rows = nullptr;  // row of the bigram table per token (hashed on the host from the previous and the current token)
    // token shift: per token the row of [h of this batch | state rows] that holds the previous token's h; per sequence of the batch its last token and its state row
    ggml_tensor *shift_src = nullptr, *shift_last = nullptr, *shift_slot = nullptr;
    // layers with convolution / recurrence state: where a token's predecessors are found, where the new state rows come from, the batch rows grouped by sequence,
    // and per sequence of the batch (first entry, count, state slot, starts here)
    ggml_tensor *seq_hist = nullptr, *seq_upd = nullptr, *seq_tok = nullptr, *seq_info = nullptr;
};

struct graph_key {
    int n_tokens = -1, n_kv = -1, n_outputs = -1, n_seqs = -1;  // n_seqs: distinct sequences of the batch (models with sequence state; else 0)
    bool operator==(const graph_key & o) const { return n_tokens == o.n_tokens && n_kv == o.n_kv && n_outputs == o.n_outputs && n_seqs == o.n_seqs; }
};

struct llm_context {
    llm_model * model = nullptr;
    ggml_backend_t backend = nullptr;
    llm_compute_fn compute = nullptr;
    llm_context_params p{};
    ggml_backend_buffer_type_t buft = nullptr;
    // KV cache
    ggml_context * ctx_kv = nullptr;
    ggml_backend_buffer_t buf_kv = nullptr;
    std::vector<ggml_tensor *> k_l, v_l;  // one pair per layer RUN (a repeated layer has a cache per pass); v is null where the values are a part of the K rows
    std::vector<kv_cell> cells;
    // sequence state of models that have it: the previous token's normed layer input per (run, sequence) — [n_embd, n_seq_max + 1, runs], the last row of a run
    // stays zero (what a sequence's first token reads) — and the previous token id per sequence (the bigram embedding's hash)
    ggml_tensor * shift_state = nullptr;
    // ... and per layer run: the last taps - 1 inputs of its short convolution [C (taps - 1), n_seq_max], the previous input of its time mixing [n_embd, n_seq_max],
    // the matrices of its recurrence [floats per sequence, n_seq_max]; all f32, null where the run has none
    std::vector<ggml_tensor *> conv_state, tm_shift_state, rec_state;
    std::vector<int32_t> seq_prev_tok;
    int n_seq_max = 0;
    std::vector<int32_t> mask_cpos, mask_cseq;  // the cells' fields as arrays (mask rows are filled from them)
    int kv_head = 0;
    int used_max = 0;           // one past the highest occupied cell; < 0: unknown (cells were freed), recounted by the next batch
    // compute graph
    ggml_gallocr_t galloc = nullptr;
    ggml_context * ctx_compute = nullptr;
    ggml_cgraph * gf = nullptr;
    graph_key key;
    ggml_tensor *inp_tokens = nullptr, *inp_pos = nullptr, *inp_mask = nullptr, *inp_k_idxs = nullptr, *inp_v_idxs = nullptr, *inp_out_ids = nullptr;
    ggml_tensor *inp_bigram = nullptr, *inp_shift_src = nullptr, *inp_shift_last = nullptr, *inp_shift_slot = nullptr;
    ggml_tensor *inp_seq_hist = nullptr, *inp_seq_upd = nullptr, *inp_seq_tok = nullptr, *inp_seq_info = nullptr;
    std::vector<ggml_tensor *> inp_masks;  // all masks of the graph (inp_masks[0] == inp_mask)
    ggml_tensor * t_logits = nullptr;
    // outputs
    std::vector<float> logits;
    float * logits_base = nullptr;  // where the last llm_decode's rows are: the pinned output area, or `logits`
    std::vector<int32_t> output_ids;  // batch position -> output row of the last llm_decode (-1: no logits requested there)
    int n_outputs = 0;
    double timings[4] = {0, 0, 0, 0};
    // pinned host staging, as llama.cpp does it (inputs are uploaded with tensor_set_async out of host-buffer-type memory,
    // logits come back with tensor_get_async into the pinned output buffer; ONE synchronize per micro-batch):
    // [ inputs of one micro-batch | logits of up to pin_out_rows outputs ]
    ggml_backend_buffer_t buf_pin = nullptr;
    char * pin = nullptr;
    size_t pin_in_bytes = 0;   // per input slot
    int pin_out_rows = 0;
    // micro-batches without outputs are not waited for (as llama.cpp: the wait happens when results are fetched); each
    // in-flight micro-batch keeps its own input slot, so the host builds and stages batch i+1 while the GPU runs batch i
    static constexpr int PIN_SLOTS = 4;
    int pin_slot = 0, in_flight = 0;
    // -sm layer (llm_context_new_layer_split): one graph segment per device, driven the way ggml_backend_sched drives the splits of a
    // layer-split model — input copies in LS_COPIES slots per device, cpy_tensor_async of the residual stream between neighbouring
    // devices, one event per (device, slot) recorded after the segment's graph and waited for before the slot is overwritten
    static constexpr int LS_COPIES = 2;
    struct ls_dev {
        ggml_backend_t be = nullptr;
        ggml_backend_buffer_type_t buft = nullptr;
        ggml_gallocr_t galloc = nullptr;
        int l0 = 0, l1 = 0;
        ggml_context * ctx_kv = nullptr;
        ggml_backend_buffer_t buf_kv = nullptr;
        ggml_context * ctx_in = nullptr;       // the input copies of all slots (+ nothing else): allocated once per graph key, outside the graph allocator
        ggml_backend_buffer_t buf_in = nullptr;
        ggml_context * ctx[LS_COPIES] = {nullptr, nullptr};
        ggml_cgraph * gf[LS_COPIES] = {nullptr, nullptr};
        seg_io io[LS_COPIES];
        ggml_backend_event_t ev[LS_COPIES] = {nullptr, nullptr};
    };
    std::vector<ls_dev> ls;
    int ls_copy = 0;
    int64_t ls_stats[4] = {0, 0, 0, 0};  // cpy_tensor_async calls between devices, blocking input copies, events recorded, events waited for
};

static ggml_tensor * named(ggml_tensor * t, const char * base, int il) {
    char buf[96];
    if (il >= 0) snprintf(buf, sizeof(buf), "%s-%d", base, il);
    else snprintf(buf, sizeof(buf), "%s", base);
    return ggml_set_name(t, buf);
}

// creates the input tensors of layers [l0, l1) (+ the output head if `head`) in `ctx`
static void make_inputs(llm_context * c, ggml_context * ctx, int l0, int l1, bool head, int n_tokens, int n_kv, int n_outputs, seg_io & io, int n_seqs = 0) {
    llm_model * m = c->model;
    const llm_hparams & hp = m->hp;
    const bool fa = c->p.flash_attn != 0;
    const int64_t n_embd_k = (int64_t) m->n_head_kv_l * hp.n_embd_head;
    io = seg_io();
    if (l0 == 0) {
        io.tokens = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, n_tokens);
        ggml_set_input(named(io.tokens, "inp_tokens", -1));
    } else {
        io.resid = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, hp.n_embd, n_tokens);
        ggml_set_input(named(io.resid, "l_out_from_the_previous_device", -1));
    }
    // (a model none of whose layers rotates has no reader of the positions: the input is then not made — the graph allocator places only what the graph reaches)
    bool need_pos = m->lcfg.empty();
    for (const llm_layer_cfg & lc : m->lcfg) need_pos = need_pos || lc.rot_dims > 0;
    if (need_pos) {
        io.pos = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, n_tokens);
        ggml_set_input(named(io.pos, "inp_pos", -1));
    }
    const int64_t n_tok_pad = (n_tokens + 63) / 64 * 64;  // GGML_KQ_MASK_PAD
    // llama.cpp's build_attn_inp_kv_unified: the mask is an F32 input filled on the host; with flash attention FLASH_ATTN_EXT is handed a
    // ggml_cast(F16) of it (self_kq_mask_cnv) — a CPY node in the graph, not an F16 upload
    if (m->has_attn) {  // (a model none of whose layers attends over the cells has no masks and no cell indices)
        io.mask = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, n_kv, n_tok_pad);
        ggml_set_input(named(io.mask, "KQ_mask", -1));
        io.masks.assign(1, io.mask);
        for (size_t k = 1; k < m->mask_rules.size(); ++k) {
            io.masks.push_back(ggml_new_tensor_2d(ctx, GGML_TYPE_F32, n_kv, n_tok_pad));
            ggml_set_input(named(io.masks.back(), "KQ_mask_chunked", (int) k));
        }
    }
    if (m->has_seq_state && m->hist_rows > 0) {  // (no layer looks back: no reader, and the graph allocator places only what the graph reaches)
        io.seq_hist = ggml_new_tensor_2d(ctx, GGML_TYPE_I32, m->hist_rows, n_tokens);
        ggml_set_input(named(io.seq_hist, "seq_hist", -1));
        io.seq_upd = ggml_new_tensor_2d(ctx, GGML_TYPE_I32, m->hist_rows, std::max(1, n_seqs));
        ggml_set_input(named(io.seq_upd, "seq_upd", -1));
    }
    if (m->has_seq_state) {
        io.seq_tok = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, n_tokens);
        ggml_set_input(named(io.seq_tok, "seq_tok", -1));
        io.seq_info = ggml_new_tensor_2d(ctx, GGML_TYPE_I32, 4, std::max(1, n_seqs));
        ggml_set_input(named(io.seq_info, "seq_info", -1));
    }
    if (m->bigram) {
        io.bigram_rows = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, n_tokens);
        ggml_set_input(named(io.bigram_rows, "inp_bigram_rows", -1));
    }
    if (m->has_shift) {
        io.shift_src = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, n_tokens);
        ggml_set_input(named(io.shift_src, "shift_src", -1));
        io.shift_last = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, std::max(1, n_seqs));
        ggml_set_input(named(io.shift_last, "shift_last_rows", -1));
        io.shift_slot = ggml_new_tensor_1d(ctx, GGML_TYPE_I64, std::max(1, n_seqs));
        ggml_set_input(named(io.shift_slot, "shift_slots", -1));
    }
    if (m->has_attn) {
        io.k_idxs = ggml_new_tensor_1d(ctx, GGML_TYPE_I64, n_tokens);
        ggml_set_input(named(io.k_idxs, "k_idxs", -1));
    }
    if (!fa) {
        io.v_idxs = ggml_new_tensor_1d(ctx, GGML_TYPE_I64, (int64_t) n_tokens * n_embd_k);
        ggml_set_input(named(io.v_idxs, "v_idxs", -1));
    }
    if (l1 == hp.n_layer && n_outputs < n_tokens) {
        io.out_ids = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, n_outputs);
        ggml_set_input(named(io.out_ids, "out_ids", -1));
    }
    (void) head;
}

// layers [l0, l1) (+ norm and output matrix if `head`) over the inputs `io`, appended to `gf`
static void build_segment(llm_context * c, ggml_context * ctx, ggml_cgraph * gf, int l0, int l1, bool head, int n_tokens, int n_kv, seg_io & io) {
    llm_model * m = c->model;
    const llm_hparams & hp = m->hp;
    const int64_t HD = hp.n_embd_head, NH = m->n_head_l, NKV = m->n_head_kv_l;
    const int64_t n_embd_k = NKV * HD, n_ctx = c->p.n_ctx;
    const bool fa = c->p.flash_attn != 0;
    const float kq_scale = 1.0f / sqrtf((float) HD);
    ggml_tensor * const mask_cnv = fa ? named(ggml_cast(ctx, io.mask, GGML_TYPE_F16), "KQ_mask_cnv", -1) : io.mask;

    ggml_tensor * inpL = l0 == 0 ? named(ggml_get_rows(ctx, m->tok_embd, io.tokens), "inp_embd", -1) : io.resid;
    for (int il = l0; il < l1; ++il) {
        const llm_layer & L = m->layers[il];
        ggml_tensor * inpSA = inpL;
        ggml_tensor * cur = named(ggml_rms_norm(ctx, inpL, hp.rms_eps), "norm", il);
        cur = named(ggml_mul(ctx, cur, L.attn_norm), "attn_norm", il);
        ggml_tensor * Qcur = named(ggml_mul_mat(ctx, L.wq, cur), "Qcur", il);
        if (L.bq) Qcur = named(ggml_add(ctx, Qcur, L.bq), "Qcur_b", il);
        ggml_tensor * Kcur = named(ggml_mul_mat(ctx, L.wk, cur), "Kcur", il);
        if (L.bk) Kcur = named(ggml_add(ctx, Kcur, L.bk), "Kcur_b", il);
        ggml_tensor * Vcur = named(ggml_mul_mat(ctx, L.wv, cur), "Vcur", il);
        if (L.bv) Vcur = named(ggml_add(ctx, Vcur, L.bv), "Vcur_b", il);
        Qcur = ggml_reshape_3d(ctx, Qcur, HD, NH, n_tokens);
        Kcur = ggml_reshape_3d(ctx, Kcur, HD, NKV, n_tokens);
        Vcur = ggml_reshape_3d(ctx, Vcur, HD, NKV, n_tokens);
        Qcur = named(ggml_rope_ext(ctx, Qcur, io.pos, nullptr, (int) HD, hp.rope_type, hp.n_ctx_train, hp.rope_freq_base, 1.0f, 0.0f, 1.0f, 32.0f, 1.0f), "Qcur_rope", il);
        Kcur = named(ggml_rope_ext(ctx, Kcur, io.pos, nullptr, (int) HD, hp.rope_type, hp.n_ctx_train, hp.rope_freq_base, 1.0f, 0.0f, 1.0f, 32.0f, 1.0f), "Kcur_rope", il);
        // llama.cpp's build_attn adds q, k and v to the graph together before the cache stores ("so that they are not reordered")
        ggml_build_forward_expand(gf, Qcur);
        ggml_build_forward_expand(gf, Kcur);
        ggml_build_forward_expand(gf, Vcur);
        // store K/V into the cache at the slots chosen for this micro-batch
        ggml_tensor * k_cache = c->k_l[il];
        ggml_tensor * v_cache = c->v_l[il];
        ggml_build_forward_expand(gf, named(ggml_set_rows(ctx, k_cache, ggml_reshape_2d(ctx, Kcur, n_embd_k, n_tokens), io.k_idxs), "k_store", il));
        if (fa) {
            ggml_build_forward_expand(gf, named(ggml_set_rows(ctx, v_cache, ggml_reshape_2d(ctx, Vcur, n_embd_k, n_tokens), io.k_idxs), "v_store", il));
        } else {
            // transposed V cache: every element is its own row of length 1
            ggml_tensor * v_view = ggml_reshape_2d(ctx, v_cache, 1, n_ctx * n_embd_k);
            ggml_tensor * v_src = ggml_reshape_2d(ctx, Vcur, 1, (int64_t) n_tokens * n_embd_k);
            ggml_build_forward_expand(gf, named(ggml_set_rows(ctx, v_view, v_src, io.v_idxs), "v_store", il));
        }
        ggml_tensor * q = ggml_permute(ctx, Qcur, 0, 2, 1, 3);  // [HD, n_tokens, NH]
        ggml_tensor * k = ggml_view_3d(ctx, k_cache, HD, n_kv, NKV, ggml_row_size(k_cache->type, n_embd_k), ggml_row_size(k_cache->type, HD), 0);
        if (fa) {
            ggml_tensor * v = ggml_view_3d(ctx, v_cache, HD, n_kv, NKV, ggml_row_size(v_cache->type, n_embd_k), ggml_row_size(v_cache->type, HD), 0);
            cur = ggml_flash_attn_ext(ctx, q, k, v, mask_cnv, kq_scale, 0.0f, 0.0f);
            ggml_flash_attn_ext_set_prec(cur, GGML_PREC_F32);
            named(cur, "fattn", il);
            cur = ggml_reshape_2d(ctx, cur, HD * NH, n_tokens);
        } else {
            ggml_tensor * v = ggml_view_3d(ctx, v_cache, n_kv, HD, NKV, ggml_row_size(v_cache->type, n_ctx), ggml_row_size(v_cache->type, n_ctx) * HD, 0);
            ggml_tensor * kq = named(ggml_mul_mat(ctx, k, q), "kq", il);  // [n_kv, n_tokens, NH]
            ggml_mul_mat_set_prec(kq, GGML_PREC_F32);
            kq = named(ggml_soft_max_ext(ctx, kq, mask_cnv, kq_scale, 0.0f), "kq_soft_max", il);
            ggml_tensor * kqv = named(ggml_mul_mat(ctx, v, kq), "kqv", il);  // [HD, n_tokens, NH]
            cur = ggml_permute(ctx, kqv, 0, 2, 1, 3);
            cur = named(ggml_cont_2d(ctx, cur, HD * NH, n_tokens), "kqv_out", il);
        }
        cur = named(ggml_mul_mat(ctx, L.wo, cur), "attn_out", il);
        if (il == hp.n_layer - 1 && io.out_ids) {
            cur = ggml_get_rows(ctx, cur, io.out_ids);
            inpSA = ggml_get_rows(ctx, inpSA, io.out_ids);
        }
        ggml_tensor * ffn_inp = named(ggml_add(ctx, cur, inpSA), "ffn_inp", il);
        cur = named(ggml_rms_norm(ctx, ffn_inp, hp.rms_eps), "norm_ffn", il);
        cur = named(ggml_mul(ctx, cur, L.ffn_norm), "ffn_norm", il);
        ggml_tensor * gate = named(ggml_mul_mat(ctx, L.ffn_gate, cur), "ffn_gate", il);
        ggml_tensor * up = named(ggml_mul_mat(ctx, L.ffn_up, cur), "ffn_up", il);
        cur = named(ggml_swiglu_split(ctx, gate, up), "ffn_swiglu", il);
        cur = named(ggml_mul_mat(ctx, L.ffn_down, cur), "ffn_out", il);
        cur = named(ggml_add(ctx, cur, ffn_inp), "l_out", il);
        inpL = cur;
    }
    ggml_tensor * cur = inpL;
    if (head) {
        cur = named(ggml_rms_norm(ctx, inpL, hp.rms_eps), "norm_final", -1);
        cur = named(ggml_mul(ctx, cur, m->output_norm), "result_norm", -1);
        cur = named(ggml_mul_mat(ctx, m->output, cur), "result_output", -1);
    }
    ggml_set_output(cur);
    ggml_build_forward_expand(gf, cur);
    io.out = cur;
}

// The graph of a model described layer by layer (llm_layer_cfg).  Per layer, with h the normed input:
//   q, k = rope(W_q h), rope(W_k h) on the leading rot_dims of every head; v = W_v h, blended with the first value-mixing layer's v;
//   k, v -> cache; attention over the cache under the layer's mask, soft-max with a sink; heads x sigmoid(W_g h); W_o; norm; + residual;
//   then the feed-forward (dense erf-GELU, or top-k experts with squared ReLU), normed before and after; + residual.
// Layer norms are NORM x weight; the residual stream and everything around the mat-muls stays f32.
static ggml_tensor * layer_norm_w(ggml_context * ctx, ggml_tensor * x, ggml_tensor * w, float eps, const char * name, int il) {
    ggml_tensor * n = named(ggml_norm(ctx, x, eps), "lnorm", il);
    return named(ggml_mul(ctx, n, w), name, il);
}

static ggml_tensor * build_moe(ggml_context * ctx, ggml_cgraph * gf, const llm_layer & L, const llm_layer_cfg & c, ggml_tensor * cur, int il) {
    const int64_t E = cur->ne[0], T = cur->ne[1];
    ggml_tensor * logits = named(ggml_mul_mat(ctx, L.ffn_gate_inp, cur), "ffn_moe_logits", il);  // [n_expert, T], f32 weights: 32-bit
    ggml_tensor * sel = named(ggml_top_k(ctx, logits, c.n_top), "ffn_moe_topk", il);            // [n_top, T] i32
    ggml_tensor * w = ggml_get_rows(ctx, ggml_reshape_3d(ctx, logits, 1, c.n_expert, T), sel);   // [1, n_top, T]
    w = named(ggml_soft_max(ctx, ggml_reshape_2d(ctx, named(w, "ffn_moe_sel_logits", il), c.n_top, T)), "ffn_moe_weights", il);  // soft-max over the chosen logits only
    ggml_tensor * up = named(ggml_mul_mat_id(ctx, L.ffn_up_exps, ggml_reshape_3d(ctx, cur, E, 1, T), sel), "ffn_moe_up", il);     // [n_ff, n_top, T]
    ggml_tensor * act = named(ggml_sqr(ctx, named(ggml_unary(ctx, up, GGML_UNARY_OP_RELU), "ffn_moe_relu", il)), "ffn_moe_act", il);
    ggml_tensor * down = named(ggml_mul_mat_id(ctx, L.ffn_down_exps, act, sel), "ffn_moe_down", il);                              // [E, n_top, T]
    down = named(ggml_mul(ctx, down, ggml_reshape_3d(ctx, w, 1, c.n_top, T)), "ffn_moe_weighted", il);
    ggml_build_forward_expand(gf, down);
    ggml_tensor * out = nullptr;
    for (int j = 0; j < c.n_top; ++j) {  // the sum over the chosen experts, as a chain of adds over views
        ggml_tensor * v = ggml_view_2d(ctx, down, E, T, down->nb[2], (size_t) j * down->nb[1]);
        out = out ? ggml_add(ctx, out, v) : v;
    }
    if (c.n_top == 1) out = ggml_cont(ctx, out);
    return named(out, "ffn_moe_out", il);
}

// the norm of a per-layer model: x / sqrt(mean(x^2) + eps) * w, or the layer norm (x - mean) / sqrt(var + eps) * w
static ggml_tensor * norm_w(ggml_context * ctx, const llm_layer_cfg & lc, ggml_tensor * x, ggml_tensor * w, float eps, const char * name, int il) {
    if (!lc.rms) return layer_norm_w(ctx, x, w, eps, name, il);
    return named(ggml_mul(ctx, named(ggml_rms_norm(ctx, x, eps), "rnorm", il), w), name, il);
}

// token shift: what the mixer reads is h + (h_prev - h) * shift, h_prev being the previous token's h — the row before it in this batch when the
// batch holds it, else the sequence's state row (a row of zeros for a sequence's first token): io.shift_src indexes [h rows | state rows].
// Afterwards every sequence's last h of the batch becomes its state row.
static ggml_tensor * build_token_shift(llm_context * c, ggml_context * ctx, ggml_cgraph * gf, ggml_tensor * h, ggml_tensor * w, int run, seg_io & io) {
    ggml_tensor * state = ggml_view_2d(ctx, c->shift_state, h->ne[0], c->shift_state->ne[1], c->shift_state->nb[1], (size_t) run * c->shift_state->nb[2]);
    ggml_tensor * both = named(ggml_concat(ctx, h, state, 1), "shift_rows", run);
    ggml_tensor * prev = named(ggml_get_rows(ctx, both, io.shift_src), "shift_prev", run);
    ggml_tensor * d = named(ggml_mul(ctx, named(ggml_sub(ctx, prev, h), "shift_diff", run), w), "shift_scaled", run);
    ggml_tensor * out = named(ggml_add(ctx, h, d), "shift_out", run);
    ggml_build_forward_expand(gf, out);  // (the state is read before it is overwritten)
    ggml_tensor * last = named(ggml_get_rows(ctx, h, io.shift_last), "shift_last", run);
    ggml_build_forward_expand(gf, named(ggml_set_rows(ctx, state, last, io.shift_slot), "shift_store", run));
    return out;
}

// grouped-query attention of one layer run over its cache; returns the heads' outputs [dv * H, T] (gated), before the output projection
static ggml_tensor * build_mixer_attention(llm_context * c, ggml_context * ctx, ggml_cgraph * gf, const llm_layer & L, const llm_layer_cfg & lc, ggml_tensor * cur, int il, int run,
                                           int n_tokens, int n_kv, seg_io & io, ggml_tensor ** v_first) {
    llm_model * m = c->model;
    const llm_hparams & hp = m->hp;
    const int64_t H = lc.n_head, G = lc.n_head_kv, DK = lc.dk, DV = lc.dv;
    (void) il;
    ggml_tensor * Qcur = named(ggml_mul_mat(ctx, L.wq, cur), "Qcur", run);
    ggml_tensor * Kcur = named(ggml_mul_mat(ctx, L.wk, cur), "Kcur", run);
    ggml_tensor * Vcur = named(ggml_mul_mat(ctx, L.wv, cur), "Vcur", run);
    ggml_tensor * gate = lc.out_gate ? named(ggml_mul_mat(ctx, L.attn_gate, cur), "attn_gate", run) : nullptr;
    if (L.bq) Qcur = named(ggml_add(ctx, Qcur, L.bq), "Qcur_b", run);
    if (L.bk) Kcur = named(ggml_add(ctx, Kcur, L.bk), "Kcur_b", run);
    if (L.bv) Vcur = named(ggml_add(ctx, Vcur, L.bv), "Vcur_b", run);
    Qcur = ggml_reshape_3d(ctx, Qcur, DK, H, n_tokens);
    Kcur = ggml_reshape_3d(ctx, Kcur, DK, G, n_tokens);
    if (lc.qk_norm) {  // every head's query and key divided by its root mean square, times a weight row shared by the heads
        Qcur = named(ggml_mul(ctx, named(ggml_rms_norm(ctx, Qcur, hp.rms_eps), "Qcur_rnorm", run), L.q_norm), "Qcur_normed", run);
        Kcur = named(ggml_mul(ctx, named(ggml_rms_norm(ctx, Kcur, hp.rms_eps), "Kcur_rnorm", run), L.k_norm), "Kcur_normed", run);
    }
    if (lc.rot_dims > 0) {  // neighbouring pairs (2i, 2i + 1) of the leading rot_dims entries; the rest of the head passes through
        Qcur = named(ggml_rope_ext(ctx, Qcur, io.pos, nullptr, lc.rot_dims, lc.rot_half ? GGML_ROPE_TYPE_NEOX : 0, hp.n_ctx_train, lc.rot_base, 1.0f, 0.0f, 1.0f, 32.0f, 1.0f), "Qcur_rope", run);
        Kcur = named(ggml_rope_ext(ctx, Kcur, io.pos, nullptr, lc.rot_dims, lc.rot_half ? GGML_ROPE_TYPE_NEOX : 0, hp.n_ctx_train, lc.rot_base, 1.0f, 0.0f, 1.0f, 32.0f, 1.0f), "Kcur_rope", run);
        ggml_rope_set_exact_freq(Qcur);  // angle = pos * base^(-2 i / dims) with the frequency itself rounded once (not ggml's running product)
        ggml_rope_set_exact_freq(Kcur);
    }
    if (lc.v_unit)  // every head's value divided by its root mean square: that is what the cache keeps
        Vcur = ggml_reshape_2d(ctx, named(ggml_rms_norm(ctx, ggml_reshape_3d(ctx, Vcur, DV, G, n_tokens), hp.rms_eps), "Vcur_unit", run), G * DV, n_tokens);
    if (lc.v_mix) {
        if (!*v_first) *v_first = Vcur;
        else {
            LLM_ASSERT((*v_first)->ne[0] == Vcur->ne[0]);
            Vcur = named(ggml_add(ctx, named(ggml_scale(ctx, Vcur, 1.0f - lc.v_lambda), "Vcur_own", run), named(ggml_scale(ctx, *v_first, lc.v_lambda), "Vcur_first", run)), "Vcur_mixed", run);
        }
    }
    ggml_build_forward_expand(gf, Qcur);
    ggml_build_forward_expand(gf, Kcur);
    ggml_build_forward_expand(gf, Vcur);
    ggml_tensor * k_cache = c->k_l[(size_t) run];
    ggml_tensor * v_cache = c->v_l[(size_t) run];
    ggml_build_forward_expand(gf, named(ggml_set_rows(ctx, k_cache, ggml_reshape_2d(ctx, Kcur, G * DK, n_tokens), io.k_idxs), "k_store", run));
    ggml_build_forward_expand(gf, named(ggml_set_rows(ctx, v_cache, ggml_reshape_2d(ctx, Vcur, G * DV, n_tokens), io.k_idxs), "v_store", run));  // (blended / normed values are what is kept)
    ggml_tensor * q = ggml_permute(ctx, Qcur, 0, 2, 1, 3);
    ggml_tensor * k = ggml_view_3d(ctx, k_cache, DK, n_kv, G, ggml_row_size(k_cache->type, G * DK), ggml_row_size(k_cache->type, DK), 0);
    ggml_tensor * v = ggml_view_3d(ctx, v_cache, DV, n_kv, G, ggml_row_size(v_cache->type, G * DV), ggml_row_size(v_cache->type, DV), 0);
    // the F32 masks go to FLASH_ATTN_EXT as they are (no F16 cast): that is how this graph asks the backend for attention in 32-bit arithmetic
    cur = ggml_flash_attn_ext(ctx, q, k, v, io.masks[(size_t) lc.mask_id], lc.scale, 0.0f, 0.0f);
    ggml_flash_attn_ext_set_prec(cur, GGML_PREC_F32);
    if (lc.sink) ggml_flash_attn_ext_add_sinks(cur, lc.sink_learned ? L.attn_sink : ggml_view_1d(ctx, m->attn_sinks, H, 0));
    if (lc.dist_pen) ggml_flash_attn_ext_add_log_distance(cur, ggml_reshape_2d(ctx, L.attn_r12, H, 2));
    named(cur, "fattn", run);
    if (gate && lc.gate_heads) {  // one number per head and token
        ggml_tensor * sg = ggml_reshape_3d(ctx, named(ggml_unary(ctx, gate, GGML_UNARY_OP_SIGMOID), "attn_gate_sigmoid", run), 1, H, n_tokens);
        cur = named(ggml_mul(ctx, cur, sg), "attn_gated", run);
        gate = nullptr;
    }
    cur = ggml_reshape_2d(ctx, cur, DV * H, n_tokens);
    if (gate) cur = named(ggml_mul(ctx, cur, named(ggml_unary(ctx, gate, GGML_UNARY_OP_SIGMOID), "attn_gate_sigmoid", run)), "attn_gated", run);
    return cur;
}

// latent attention of one layer run.  The cache row of a token is [c | k_r]: the normed latent (kv_rank values) and the rotated key part shared by all
// heads.  Keys and values are never expanded: with k_h = W_uk,h c the score q_h . k_h equals (W_uk,h^T q_h) . c, so the query is taken into the latent
// space (one small mat-mul per head), every head attends over the SAME rows [c | k_r] with the query [W_uk,h^T q_h | rot(q_r,h)], the weighted sum of
// the latents comes back, and W_uv,h expands it to the head's value.  Returns [dv * H, T].
static ggml_tensor * build_mixer_latent(llm_context * c, ggml_context * ctx, ggml_cgraph * gf, const llm_layer & L, const llm_layer_cfg & lc, ggml_tensor * cur, int il, int run,
                                        int n_tokens, int n_kv, seg_io & io) {
    llm_model * m = c->model;
    const llm_hparams & hp = m->hp;
    const int64_t H = lc.n_head, DK = lc.dk, DR = lc.rot_dim, DV = lc.dv, R = lc.kv_rank, DQ = DK + DR, ROW = R + DR;
    const float mag = rope_magnitude(lc);
    (void) il;
    const int rope_mode = lc.rot_half ? GGML_ROPE_TYPE_NEOX : 0;  // pairs (i, i + dr / 2), or neighbours (2i, 2i + 1)
    const bool own_rows = lc.kv_from < 0;                        // (else: the rows another layer's cache holds — no down projection, nothing stored)
    // the projections of the one input follow one another: the query (or its latent), the latent of keys and values, the output gate
    ggml_tensor * q_in = cur;
    ggml_tensor * q_lat_pre = L.wdq ? named(ggml_mul_mat(ctx, L.wdq, cur), "q_a", run) : nullptr;
    ggml_tensor * ckr = own_rows ? named(ggml_mul_mat(ctx, L.wdkv, cur), "kv_a", run) : nullptr;  // [R + DR, T]
    ggml_tensor * gate = lc.out_gate ? named(ggml_mul_mat(ctx, L.attn_gate, cur), "attn_gate", run) : nullptr;
    if (q_lat_pre) {
        ggml_build_forward_expand(gf, q_lat_pre);
        if (ckr) ggml_build_forward_expand(gf, ckr);
        if (gate) ggml_build_forward_expand(gf, gate);
        q_in = named(ggml_mul(ctx, named(ggml_rms_norm(ctx, q_lat_pre, hp.rms_eps), "q_a_rnorm", run), L.dq_norm), "q_latent_normed", run);  // the queries' own normed latent
    }
    ggml_tensor * Qcur = named(ggml_mul_mat(ctx, L.wq, q_in), "Qcur", run);        // [DQ * H, T]: head by head [dk unrotated | dr rotated]
    int cache_run = run;
    if (!own_rows) {
        cache_run = -1;
        for (int r = 0; r < run; ++r)
            if (m->runs[(size_t) r].il == lc.kv_from && m->runs[(size_t) r].pass == m->runs[(size_t) run].pass) cache_run = r;
        LLM_ASSERT(cache_run >= 0 && c->k_l[(size_t) cache_run]);
    }
    ggml_tensor * k_cache = c->k_l[(size_t) cache_run];
    ggml_tensor * q_rot = nullptr;
    if (DR > 0) {
        q_rot = ggml_view_3d(ctx, Qcur, DR, H, n_tokens, (size_t) DQ * sizeof(float), Qcur->nb[1], (size_t) DK * sizeof(float));
        q_rot = named(ggml_rope_ext(ctx, q_rot, io.pos, L.rope_freq, (int) DR, rope_mode, hp.n_ctx_train, lc.rot_base, 1.0f, 0.0f, mag, 32.0f, 1.0f), "q_rot", run);
        ggml_rope_set_freq_table(q_rot);
    }
    if (own_rows) {
        ggml_tensor * lat = ggml_view_2d(ctx, ckr, R, n_tokens, ckr->nb[1], 0);
        lat = named(ggml_mul(ctx, named(ggml_rms_norm(ctx, lat, hp.rms_eps), "kv_a_rnorm", run), L.dkv_norm), "kv_latent", run);
        ggml_tensor * krow = lat;
        if (DR > 0) {
            ggml_tensor * kr = ggml_view_3d(ctx, ckr, DR, 1, n_tokens, ckr->nb[1], ckr->nb[1], (size_t) R * sizeof(float));
            kr = named(ggml_rope_ext(ctx, kr, io.pos, L.rope_freq, (int) DR, rope_mode, hp.n_ctx_train, lc.rot_base, 1.0f, 0.0f, mag, 32.0f, 1.0f), "k_rot", run);
            ggml_rope_set_freq_table(kr);
            krow = named(ggml_concat(ctx, lat, ggml_reshape_2d(ctx, kr, DR, n_tokens), 0), "kv_row", run);
        }
        ggml_build_forward_expand(gf, krow);
        ggml_build_forward_expand(gf, named(ggml_set_rows(ctx, k_cache, krow, io.k_idxs), "kv_store", run));
    }
    // the unrotated part of every head's query, [dk, T, H] seen through strides, times W_uk,h^T -> [R, T, H]
    ggml_tensor * q_nope = ggml_view_3d(ctx, Qcur, DK, n_tokens, H, Qcur->nb[1], (size_t) DQ * sizeof(float), 0);
    ggml_tensor * q_lat = named(ggml_mul_mat(ctx, L.wuk_t, q_nope), "q_latent", run);
    ggml_tensor * q = ggml_permute(ctx, q_lat, 0, 2, 1, 3);  // [R, H, T]
    if (q_rot) q = named(ggml_concat(ctx, q, q_rot, 0), "q_row", run);  // [R + DR, H, T]
    else q = named(ggml_cont(ctx, q), "q_row", run);
    ggml_tensor * k = ggml_view_3d(ctx, k_cache, ROW, n_kv, 1, ggml_row_size(k_cache->type, ROW), ggml_row_size(k_cache->type, ROW), 0);
    ggml_tensor * v = ggml_view_3d(ctx, k_cache, R, n_kv, 1, ggml_row_size(k_cache->type, ROW), ggml_row_size(k_cache->type, ROW), 0);  // the latent part of the same rows
    ggml_tensor * att = ggml_flash_attn_ext(ctx, ggml_permute(ctx, q, 0, 2, 1, 3), k, v, io.masks[(size_t) lc.mask_id], lc.scale, 0.0f, 0.0f);  // [R, H, T]
    ggml_flash_attn_ext_set_prec(att, GGML_PREC_F32);
    if (lc.sink) ggml_flash_attn_ext_add_sinks(att, lc.sink_learned ? L.attn_sink : ggml_view_1d(ctx, m->attn_sinks, H, 0));
    named(att, "fattn", run);
    ggml_tensor * o = named(ggml_mul_mat(ctx, L.wuv, ggml_permute(ctx, att, 0, 2, 1, 3)), "v_expand", run);  // [DV, T, H]
    o = named(ggml_cont_2d(ctx, ggml_permute(ctx, o, 0, 2, 1, 3), DV * H, n_tokens), "attn_heads", run);
    if (gate) o = named(ggml_mul(ctx, o, named(ggml_unary(ctx, gate, GGML_UNARY_OP_SIGMOID), "attn_gate_sigmoid", run)), "attn_gated", run);  // one gate per value entry
    return o;
}

// ---- mixers with state per sequence.  Each returns the mixer's output [n_embd, T] (its own output projection included).
// the per-head norm behind a recurrence: every head's o divided by its root mean square, times a weight (one row shared by the heads, or one entry per (head, entry)),
// times an activation of the gate projection
static ggml_tensor * build_head_norm_gate(ggml_context * ctx, ggml_tensor * o, ggml_tensor * w, ggml_tensor * gate, enum ggml_unary_op act, float eps, int run) {
    const int64_t DV = o->ne[0], H = o->ne[1], T = o->ne[2];
    ggml_tensor * n = named(ggml_rms_norm(ctx, o, eps), "head_rnorm", run);
    if (ggml_nelements(w) == DV) n = named(ggml_mul(ctx, n, w), "head_norm", run);
    else n = named(ggml_mul(ctx, n, ggml_reshape_2d(ctx, w, DV, H)), "head_norm", run);
    n = ggml_reshape_2d(ctx, n, DV * H, T);
    return named(ggml_mul(ctx, n, named(ggml_unary(ctx, gate, act), "head_gate_act", run)), "head_gated", run);
}

static ggml_tensor * build_mixer_mlstm(llm_context * c, ggml_context * ctx, ggml_cgraph * gf, const llm_layer & L, const llm_layer_cfg & lc, ggml_tensor * cur, int run, int n_tokens, seg_io & io) {
    const int64_t H = lc.n_head, DK = lc.dk, DV = lc.dv;
    ggml_tensor * qkv = named(ggml_mul_mat(ctx, L.wqkv, cur), "qkv", run);
    ggml_tensor * gates = named(ggml_mul_mat(ctx, L.wgates, cur), "if_pre", run);
    ggml_tensor * gate = named(ggml_mul_mat(ctx, L.attn_gate, cur), "attn_gate", run);
    ggml_build_forward_expand(gf, qkv);  // (the three products of the one input follow one another)
    ggml_build_forward_expand(gf, gates);
    ggml_build_forward_expand(gf, gate);
    ggml_tensor * q = ggml_view_2d(ctx, qkv, H * DK, n_tokens, qkv->nb[1], 0);
    ggml_tensor * k = ggml_view_2d(ctx, qkv, H * DK, n_tokens, qkv->nb[1], (size_t) (H * DK) * sizeof(float));
    ggml_tensor * v = ggml_view_2d(ctx, qkv, H * DV, n_tokens, qkv->nb[1], (size_t) (2 * H * DK) * sizeof(float));
    ggml_tensor * o = named(ggml_seq_mlstm(ctx, q, k, v, gates, L.gate_par, c->rec_state[(size_t) run], io.seq_tok, io.seq_info, (int) H, lc.gate_cap), "mlstm", run);
    cur = build_head_norm_gate(ctx, o, L.sub_norm, gate, GGML_UNARY_OP_SIGMOID, c->model->hp.rms_eps, run);
    return named(ggml_mul_mat(ctx, L.wo, cur), "attn_out", run);
}

static ggml_tensor * build_mixer_delta(llm_context * c, ggml_context * ctx, ggml_cgraph * gf, const llm_layer & L, const llm_layer_cfg & lc, ggml_tensor * cur, int run, int n_tokens, seg_io & io) {
    const int64_t H = lc.n_head, G = lc.n_head_kv, DK = lc.dk, DV = lc.dv;
    ggml_tensor * qkv_pre = named(ggml_mul_mat(ctx, L.wqkv, cur), "qkv_pre", run);
    ggml_tensor * gates = named(ggml_mul_mat(ctx, L.wgates, cur), "ba_pre", run);
    ggml_tensor * gate = named(ggml_mul_mat(ctx, L.attn_gate, cur), "attn_gate", run);
    ggml_build_forward_expand(gf, qkv_pre);  // (the three products of the one input follow one another)
    ggml_build_forward_expand(gf, gates);
    ggml_build_forward_expand(gf, gate);
    ggml_tensor * qkv = named(ggml_seq_conv(ctx, qkv_pre, L.conv, c->conv_state[(size_t) run], io.seq_hist, /*act=*/1), "qkv_conv", run);
    ggml_build_forward_expand(gf, qkv);  // (the state is read before it is overwritten)
    if (lc.conv_taps > 1) ggml_build_forward_expand(gf, named(ggml_seq_conv_store(ctx, c->conv_state[(size_t) run], qkv_pre, io.seq_upd, io.seq_info, lc.conv_taps), "conv_store", run));
    qkv = ggml_reshape_2d(ctx, qkv, qkv->ne[0], n_tokens);
    ggml_tensor * q = ggml_view_2d(ctx, qkv, G * DK, n_tokens, qkv->nb[1], 0);
    ggml_tensor * k = ggml_view_2d(ctx, qkv, G * DK, n_tokens, qkv->nb[1], (size_t) (G * DK) * sizeof(float));
    ggml_tensor * v = ggml_view_2d(ctx, qkv, H * DV, n_tokens, qkv->nb[1], (size_t) (2 * G * DK) * sizeof(float));
    ggml_tensor * o = named(ggml_seq_gated_delta(ctx, q, k, v, gates, L.gate_par, c->rec_state[(size_t) run], io.seq_tok, io.seq_info, (int) H, (int) G), "gated_delta", run);
    cur = build_head_norm_gate(ctx, o, L.sub_norm, gate, GGML_UNARY_OP_SILU, c->model->hp.rms_eps, run);
    return named(ggml_mul_mat(ctx, L.wo, cur), "attn_out", run);
}

// windowed sigmoid attention (left) and time mixing (right) over the same input; the mixer is left_scale * left + right_scale * right
static ggml_tensor * build_mixer_sigmoid_wkv(llm_context * c, ggml_context * ctx, ggml_cgraph * gf, const llm_layer & L, const llm_layer_cfg & lc, ggml_tensor * cur, int run, int n_tokens,
                                             int n_kv, seg_io & io) {
    llm_model * m = c->model;
    const llm_hparams & hp = m->hp;
    const int64_t H = lc.n_head, G = lc.n_head_kv, DK = lc.dk, DV = lc.dv, E = hp.n_embd;
    // ---- left: projection (+ bias) -> short convolution -> rotation of q and k -> cache -> attention with sigmoid weights
    ggml_tensor * qkv_pre = named(ggml_mul_mat(ctx, L.wqkv, cur), "qkv_proj", run);
    if (L.bqkv) qkv_pre = named(ggml_add(ctx, qkv_pre, L.bqkv), "qkv_pre", run);
    ggml_tensor * qkv = named(ggml_seq_conv(ctx, qkv_pre, L.conv, c->conv_state[(size_t) run], io.seq_hist, /*act=*/0), "qkv_conv", run);
    ggml_build_forward_expand(gf, qkv);
    if (lc.conv_taps > 1) ggml_build_forward_expand(gf, named(ggml_seq_conv_store(ctx, c->conv_state[(size_t) run], qkv_pre, io.seq_upd, io.seq_info, lc.conv_taps), "conv_store", run));
    qkv = ggml_reshape_2d(ctx, qkv, qkv->ne[0], n_tokens);
    ggml_tensor * Qcur = ggml_view_3d(ctx, qkv, DK, H, n_tokens, (size_t) DK * sizeof(float), qkv->nb[1], 0);
    ggml_tensor * Kcur = ggml_view_3d(ctx, qkv, DK, G, n_tokens, (size_t) DK * sizeof(float), qkv->nb[1], (size_t) (H * DK) * sizeof(float));
    ggml_tensor * Vcur = ggml_view_2d(ctx, qkv, G * DV, n_tokens, qkv->nb[1], (size_t) ((H + G) * DK) * sizeof(float));
    if (lc.rot_dims > 0) {
        Qcur = named(ggml_rope_ext(ctx, Qcur, io.pos, nullptr, lc.rot_dims, GGML_ROPE_TYPE_NEOX, hp.n_ctx_train, lc.rot_base, 1.0f, 0.0f, 1.0f, 32.0f, 1.0f), "Qcur_rope", run);
        Kcur = named(ggml_rope_ext(ctx, Kcur, io.pos, nullptr, lc.rot_dims, GGML_ROPE_TYPE_NEOX, hp.n_ctx_train, lc.rot_base, 1.0f, 0.0f, 1.0f, 32.0f, 1.0f), "Kcur_rope", run);
        ggml_rope_set_exact_freq(Qcur);
        ggml_rope_set_exact_freq(Kcur);
    } else {
        Qcur = named(ggml_cont(ctx, Qcur), "Qcur_cont", run);
        Kcur = named(ggml_cont(ctx, Kcur), "Kcur_cont", run);
    }
    ggml_build_forward_expand(gf, Qcur);
    ggml_build_forward_expand(gf, Kcur);
    ggml_build_forward_expand(gf, Vcur);
    ggml_tensor * k_cache = c->k_l[(size_t) run];
    ggml_tensor * v_cache = c->v_l[(size_t) run];
    ggml_build_forward_expand(gf, named(ggml_set_rows(ctx, k_cache, ggml_reshape_2d(ctx, Kcur, G * DK, n_tokens), io.k_idxs), "k_store", run));
    ggml_build_forward_expand(gf, named(ggml_set_rows(ctx, v_cache, Vcur, io.k_idxs), "v_store", run));
    ggml_tensor * qp = ggml_permute(ctx, Qcur, 0, 2, 1, 3);
    ggml_tensor * kc = ggml_view_3d(ctx, k_cache, DK, n_kv, G, ggml_row_size(k_cache->type, G * DK), ggml_row_size(k_cache->type, DK), 0);
    ggml_tensor * vc = ggml_view_3d(ctx, v_cache, DV, n_kv, G, ggml_row_size(v_cache->type, G * DV), ggml_row_size(v_cache->type, DV), 0);
    ggml_tensor * att = ggml_flash_attn_ext(ctx, qp, kc, vc, io.masks[(size_t) lc.mask_id], lc.scale, 0.0f, lc.softcap);
    ggml_flash_attn_ext_set_prec(att, GGML_PREC_F32);
    ggml_flash_attn_ext_set_sigmoid(att, L.attn_fb);
    named(att, "fattn", run);
    ggml_tensor * left = named(ggml_mul_mat(ctx, L.wo, ggml_reshape_2d(ctx, att, DV * H, n_tokens)), "attn_out", run);
    if (L.bo) left = named(ggml_add(ctx, left, L.bo), "attn_out_b", run);
    // ---- right: five token-shifted copies of the input (2-tap convolutions over the sequence) -> r, k, v, gate and the decay -> the recurrence -> norm, gate, projection
    const int64_t TH = lc.tm_heads, TD = lc.tm_dim, D = TH * TD;
    ggml_tensor * mix = named(ggml_seq_conv(ctx, cur, L.tm_taps, c->tm_shift_state[(size_t) run], io.seq_hist, 0), "time_mix_in", run);  // [E, T, 5]
    ggml_build_forward_expand(gf, mix);
    ggml_build_forward_expand(gf, named(ggml_seq_conv_store(ctx, c->tm_shift_state[(size_t) run], cur, io.seq_upd, io.seq_info, 2), "time_mix_store", run));
    ggml_tensor * mix4 = ggml_view_3d(ctx, mix, E, n_tokens, 4, mix->nb[1], mix->nb[2], 0);
    ggml_tensor * rkvg = named(ggml_mul_mat(ctx, L.tm_rkvg, mix4), "time_mix_rkvg", run);  // [D, T, 4]
    ggml_tensor * mixw = ggml_view_2d(ctx, mix, E, n_tokens, mix->nb[1], 4 * mix->nb[2]);
    ggml_tensor * wl = named(ggml_unary(ctx, named(ggml_mul_mat(ctx, L.tm_w1, mixw), "time_mix_w1", run), GGML_UNARY_OP_TANH), "time_mix_w1_tanh", run);
    ggml_tensor * w_pre = named(ggml_mul_mat(ctx, L.tm_w2, wl), "time_mix_w_pre", run);  // [D, T]
    ggml_tensor * r = ggml_view_2d(ctx, rkvg, D, n_tokens, rkvg->nb[1], 0);
    ggml_tensor * k = ggml_view_2d(ctx, rkvg, D, n_tokens, rkvg->nb[1], rkvg->nb[2]);
    ggml_tensor * v = ggml_view_2d(ctx, rkvg, D, n_tokens, rkvg->nb[1], 2 * rkvg->nb[2]);
    ggml_tensor * g = ggml_view_2d(ctx, rkvg, D, n_tokens, rkvg->nb[1], 3 * rkvg->nb[2]);
    ggml_tensor * o = named(ggml_seq_wkv6(ctx, r, k, v, w_pre, L.tm_w0, L.tm_u, c->rec_state[(size_t) run], io.seq_tok, io.seq_info, (int) TH), "wkv6", run);
    ggml_tensor * gated = build_head_norm_gate(ctx, o, L.tm_norm, g, GGML_UNARY_OP_SILU, hp.rms_eps, run);
    ggml_tensor * right = named(ggml_mul_mat(ctx, L.tm_out, gated), "time_mix_out", run);
    ggml_build_forward_expand(gf, left);
    ggml_build_forward_expand(gf, right);  // (both branches first: the two SCALEs and their ADD then follow one another, which the backend runs as one blend)
    return named(ggml_add(ctx, named(ggml_scale(ctx, left, lc.left_scale), "mix_left", run), named(ggml_scale(ctx, right, lc.right_scale), "mix_right", run)), "mix_sum", run);
}

// state-space duality (Mamba-2): the input projection in three parts — the gate z, (x, B, C) through a short convolution with bias and SiLU, the step sizes —, the
// recurrence per head over a state of N x dv, y times silu(z), an RMS norm over equal parts of the row, the output projection
static ggml_tensor * build_mixer_ssd(llm_context * c, ggml_context * ctx, ggml_cgraph * gf, const llm_layer & L, const llm_layer_cfg & lc, ggml_tensor * cur, int run, int n_tokens, seg_io & io) {
    const int64_t H = lc.n_head, DV = lc.dv, N = lc.ssm_state, G = lc.ssm_groups, inner = H * DV, GN = G * N, NG = lc.ssm_norm_groups;
    ggml_tensor * z = named(ggml_mul_mat(ctx, L.ssm_in_z, cur), "ssm_z", run);
    ggml_tensor * xbc_pre = named(ggml_mul_mat(ctx, L.ssm_in_xbc, cur), "ssm_xbc_pre", run);
    ggml_tensor * dt = named(ggml_mul_mat(ctx, L.ssm_in_dt, cur), "ssm_dt_pre", run);
    ggml_build_forward_expand(gf, z);  // (the three products of the one input follow one another)
    ggml_build_forward_expand(gf, xbc_pre);
    ggml_build_forward_expand(gf, dt);
    ggml_tensor * xbc = named(ggml_seq_conv(ctx, xbc_pre, L.conv, c->conv_state[(size_t) run], io.seq_hist, /*act=*/1), "ssm_xbc", run);
    if (L.conv_b) ggml_seq_conv_set_bias(xbc, L.conv_b);
    ggml_build_forward_expand(gf, xbc);  // (the state is read before it is overwritten)
    if (lc.conv_taps > 1) ggml_build_forward_expand(gf, named(ggml_seq_conv_store(ctx, c->conv_state[(size_t) run], xbc_pre, io.seq_upd, io.seq_info, lc.conv_taps), "conv_store", run));
    xbc = ggml_reshape_2d(ctx, xbc, xbc->ne[0], n_tokens);
    ggml_tensor * x = ggml_view_2d(ctx, xbc, inner, n_tokens, xbc->nb[1], 0);
    ggml_tensor * B = ggml_view_2d(ctx, xbc, GN, n_tokens, xbc->nb[1], (size_t) inner * sizeof(float));
    ggml_tensor * C = ggml_view_2d(ctx, xbc, GN, n_tokens, xbc->nb[1], (size_t) (inner + GN) * sizeof(float));
    ggml_tensor * y = named(ggml_seq_ssd(ctx, C, B, x, dt, L.gate_par, c->rec_state[(size_t) run], io.seq_tok, io.seq_info, (int) H, (int) G), "ssd", run);  // [DV, H, T]
    // the gate comes before the norm
    y = named(ggml_mul(ctx, ggml_reshape_2d(ctx, y, inner, n_tokens), named(ggml_unary(ctx, z, GGML_UNARY_OP_SILU), "ssm_z_silu", run)), "ssm_gated", run);
    y = named(ggml_rms_norm(ctx, ggml_reshape_3d(ctx, y, inner / NG, NG, n_tokens), c->model->hp.rms_eps), "ssm_rnorm", run);
    y = named(ggml_mul(ctx, y, ggml_reshape_2d(ctx, L.sub_norm, inner / NG, NG)), "ssm_normed", run);
    return named(ggml_mul_mat(ctx, L.wo, ggml_reshape_2d(ctx, y, inner, n_tokens)), "attn_out", run);
}

// a gated delta rule with one decay per (head, key channel): q, k, v as one projection through short convolutions + SiLU; beta; the decay's and the output gate's
// raw values through two small matrices each; the recurrence; per-head norm x weight x sigmoid(gate); `wo`.  Returns [n_embd, T]
static ggml_tensor * build_mixer_delta_channel(llm_context * c, ggml_context * ctx, ggml_cgraph * gf, const llm_layer & L, ggml_tensor * wo, int H, int G, int DK, int DV, int taps,
                                               ggml_tensor * cur, int run, int n_tokens, seg_io & io) {
    ggml_tensor * qkv_pre = named(ggml_mul_mat(ctx, L.wqkv, cur), "delta_qkv_pre", run);
    ggml_tensor * b_pre = named(ggml_mul_mat(ctx, L.wbeta, cur), "delta_b_pre", run);
    ggml_tensor * a_in = named(ggml_mul_mat(ctx, L.wa1, cur), "delta_a_in", run);
    ggml_tensor * g_in = named(ggml_mul_mat(ctx, L.wg1, cur), "delta_g_in", run);
    ggml_build_forward_expand(gf, qkv_pre);  // (the products of the one input follow one another)
    ggml_build_forward_expand(gf, b_pre);
    ggml_build_forward_expand(gf, a_in);
    ggml_build_forward_expand(gf, g_in);
    ggml_tensor * a_pre = named(ggml_mul_mat(ctx, L.wa2, a_in), "delta_a_pre", run);  // [DK H, T]
    ggml_tensor * gate = named(ggml_mul_mat(ctx, L.wg2, g_in), "delta_gate", run);    // [DV H, T]
    ggml_build_forward_expand(gf, a_pre);
    ggml_build_forward_expand(gf, gate);
    ggml_tensor * qkv = named(ggml_seq_conv(ctx, qkv_pre, L.conv, c->conv_state[(size_t) run], io.seq_hist, /*act=*/1), "delta_qkv", run);
    ggml_build_forward_expand(gf, qkv);  // (the state is read before it is overwritten)
    if (taps > 1) ggml_build_forward_expand(gf, named(ggml_seq_conv_store(ctx, c->conv_state[(size_t) run], qkv_pre, io.seq_upd, io.seq_info, taps), "conv_store", run));
    qkv = ggml_reshape_2d(ctx, qkv, qkv->ne[0], n_tokens);
    ggml_tensor * q = ggml_view_2d(ctx, qkv, (int64_t) G * DK, n_tokens, qkv->nb[1], 0);
    ggml_tensor * k = ggml_view_2d(ctx, qkv, (int64_t) G * DK, n_tokens, qkv->nb[1], (size_t) (G * DK) * sizeof(float));
    ggml_tensor * v = ggml_view_2d(ctx, qkv, (int64_t) H * DV, n_tokens, qkv->nb[1], (size_t) (2 * G * DK) * sizeof(float));
    ggml_tensor * o = named(ggml_seq_delta_channel(ctx, q, k, v, b_pre, a_pre, L.gate_par, c->rec_state[(size_t) run], io.seq_tok, io.seq_info, H, G), "delta_channel", run);
    cur = build_head_norm_gate(ctx, o, L.sub_norm, gate, GGML_UNARY_OP_SIGMOID, c->model->hp.rms_eps, run);
    return named(ggml_mul_mat(ctx, wo, cur), "delta_out", run);
}

// grouped-query attention (left) and the delta rule with channel decay (right) over the same input; each output is RMS-normed over the width with a weight of its own,
// and the mixer is left_scale * left + right_scale * right
static ggml_tensor * build_mixer_attn_delta(llm_context * c, ggml_context * ctx, ggml_cgraph * gf, const llm_layer & L, const llm_layer_cfg & lc, ggml_tensor * cur, int il, int run,
                                            int n_tokens, int n_kv, seg_io & io) {
    const float eps = c->model->hp.rms_eps;
    ggml_tensor * v_first = nullptr;
    ggml_tensor * left = build_mixer_attention(c, ctx, gf, L, lc, cur, il, run, n_tokens, n_kv, io, &v_first);
    left = named(ggml_mul_mat(ctx, L.wo, left), "attn_out", run);
    ggml_build_forward_expand(gf, left);
    ggml_tensor * right = build_mixer_delta_channel(c, ctx, gf, L, L.wo_r, lc.r_head, lc.r_head_kv, lc.r_dk, lc.r_dv, lc.conv_taps, cur, run, n_tokens, io);
    ggml_build_forward_expand(gf, right);  // (both branches first: the two norms, the two SCALEs and their ADD then follow one another, which the backend runs as one launch)
    left = named(ggml_mul(ctx, named(ggml_rms_norm(ctx, left, eps), "mix_left_rnorm", run), L.left_norm), "mix_left_normed", run);
    right = named(ggml_mul(ctx, named(ggml_rms_norm(ctx, right, eps), "mix_right_rnorm", run), L.right_norm), "mix_right_normed", run);
    return named(ggml_add(ctx, named(ggml_scale(ctx, left, lc.left_scale), "mix_left", run), named(ggml_scale(ctx, right, lc.right_scale), "mix_right", run)), "mix_sum", run);
}

// the per-layer token input: e = the layer's row of the side table for every token; x += rms_norm(W_proj (gelu_tanh(W_gate x) * e)) * w
static ggml_tensor * build_token_side(ggml_context * ctx, const llm_layer & L, ggml_tensor * x, ggml_tensor * e, float eps, int run) {
    ggml_tensor * g = named(ggml_unary(ctx, named(ggml_mul_mat(ctx, L.side_gate, x), "side_gate", run), GGML_UNARY_OP_GELU), "side_gelu", run);
    g = named(ggml_mul(ctx, g, e), "side_gated", run);
    ggml_tensor * y = named(ggml_mul_mat(ctx, L.side_proj, g), "side_proj", run);
    y = named(ggml_mul(ctx, named(ggml_rms_norm(ctx, y, eps), "side_rnorm", run), L.side_norm), "side_normed", run);
    return named(ggml_add(ctx, x, y), "l_out_side", run);
}

// experts chosen by a soft-max over ALL experts, confined to the best groups; weights = chosen scores x scale; experts W_down (silu(W_gate h) * W_up h)
static ggml_tensor * build_moe_grouped(ggml_context * ctx, ggml_cgraph * gf, const llm_layer & L, const llm_layer_cfg & c, ggml_tensor * cur, int il) {
    const int64_t E = cur->ne[0], T = cur->ne[1], FF = c.n_ff;
    ggml_tensor * logits = named(ggml_mul_mat(ctx, L.ffn_gate_inp, cur), "ffn_moe_logits", il);  // [n_expert, T], f32 weights: 32-bit
    ggml_tensor * probs = named(ggml_soft_max(ctx, logits), "ffn_moe_probs", il);
    ggml_tensor * order = c.moe_groups > 1 && c.moe_keep < c.moe_groups ? ggml_argsort_grouped(ctx, probs, c.moe_groups, c.moe_keep) : ggml_argsort(ctx, probs, 1);
    named(order, "ffn_moe_order", il);
    ggml_tensor * sel = ggml_view_2d(ctx, order, c.n_top, T, order->nb[1], 0);  // [n_top, T] i32
    ggml_tensor * w = named(ggml_get_rows(ctx, ggml_reshape_3d(ctx, probs, 1, c.n_expert, T), sel), "ffn_moe_sel_probs", il);  // [1, n_top, T]
    w = named(ggml_scale(ctx, w, c.moe_scale), "ffn_moe_weights", il);
    ggml_build_forward_expand(gf, w);  // (the weights before the experts' products: the router is then one run of nodes, which the backend takes as one launch)
    ggml_tensor * gu = named(ggml_mul_mat_id(ctx, L.ffn_gate_up_exps, ggml_reshape_3d(ctx, cur, E, 1, T), sel), "ffn_moe_gate_up", il);  // [2 ff, n_top, T]: gate rows, then up rows
    ggml_tensor * act = named(ggml_swiglu(ctx, ggml_reshape_2d(ctx, gu, 2 * FF, c.n_top * T)), "ffn_moe_act", il);                        // [ff, n_top T]
    ggml_tensor * down = named(ggml_mul_mat_id(ctx, L.ffn_down_exps, ggml_reshape_3d(ctx, act, FF, c.n_top, T), sel), "ffn_moe_down", il);  // [E, n_top, T]
    down = named(ggml_mul(ctx, down, w), "ffn_moe_weighted", il);
    ggml_build_forward_expand(gf, down);
    ggml_tensor * out = nullptr;
    for (int j = 0; j < c.n_top; ++j) {
        ggml_tensor * v = ggml_view_2d(ctx, down, E, T, down->nb[2], (size_t) j * down->nb[1]);
        out = out ? ggml_add(ctx, out, v) : v;
    }
    if (c.n_top == 1) out = ggml_cont(ctx, out);
    return named(out, "ffn_moe_out", il);
}

static ggml_tensor * build_ffn(ggml_context * ctx, ggml_cgraph * gf, const llm_layer & L, const llm_layer_cfg & lc, ggml_tensor * cur, int il, int run) {
    if (lc.mlp == LLM_MLP_MOE) return lc.moe_scores_all ? build_moe_grouped(ctx, gf, L, lc, cur, il) : build_moe(ctx, gf, L, lc, cur, il);
    if (lc.ffn_gated_tanh) {
        ggml_tensor * g = named(ggml_add(ctx, named(ggml_mul_mat(ctx, L.ffn_gate, cur), "ffn_gate", run), L.ffn_gate_b), "ffn_gate_b", run);
        ggml_tensor * u = named(ggml_add(ctx, named(ggml_mul_mat(ctx, L.ffn_up, cur), "ffn_up", run), L.ffn_up_b), "ffn_up_b", run);
        cur = named(ggml_mul(ctx, named(ggml_unary(ctx, g, GGML_UNARY_OP_GELU), "ffn_gelu", run), u), "ffn_act", run);
        return named(ggml_add(ctx, named(ggml_mul_mat(ctx, L.ffn_down, cur), "ffn_down", run), L.ffn_down_b), "ffn_out", run);
    }
    cur = named(ggml_mul_mat(ctx, L.ffn_up, cur), "ffn_up", run);
    if (lc.ffn_relu_sq) cur = named(ggml_sqr(ctx, named(ggml_unary(ctx, cur, GGML_UNARY_OP_RELU), "ffn_relu", run)), "ffn_act", run);
    else cur = named(ggml_unary(ctx, cur, GGML_UNARY_OP_GELU_ERF), "ffn_gelu", run);
    return named(ggml_mul_mat(ctx, L.ffn_down, cur), "ffn_out", run);
}

static void build_layerwise(llm_context * c, ggml_context * ctx, ggml_cgraph * gf, int n_tokens, int n_kv, seg_io & io) {
    llm_model * m = c->model;
    const llm_hparams & hp = m->hp;
    const float eps = hp.rms_eps;
    ggml_tensor * inpL = named(ggml_get_rows(ctx, m->tok_embd, io.tokens), "inp_embd", -1);
    if (m->embd_scale != 1.0f) inpL = named(ggml_scale(ctx, inpL, m->embd_scale), "inp_scaled", -1);
    if (m->bigram) inpL = named(ggml_add(ctx, inpL, named(ggml_get_rows(ctx, m->bigram, io.bigram_rows), "inp_bigram", -1)), "inp_sum", -1);
    ggml_tensor * const embd_out = inpL;
    ggml_tensor * v_first = nullptr;
    const int n_runs = (int) m->runs.size();
    for (int run = 0; run < n_runs; ++run) {
        const int il = m->runs[(size_t) run].il;
        const llm_layer & L = m->layers[(size_t) il];
        const llm_layer_cfg & lc = m->lcfg[(size_t) il];
        const bool last = run == n_runs - 1;
        if (m->runs[(size_t) run].first) {  // a pass through the repeated range begins: x <- W_in [x; embedding output] + step[pass] (without W_in: x + embedding output
                                            // from the second pass on, + step[pass])
            if (m->loop_in) inpL = named(ggml_mul_mat(ctx, m->loop_in, named(ggml_concat(ctx, inpL, embd_out, 0), "loop_cat", run)), "loop_in", run);
            else if (m->runs[(size_t) run].pass > 0) inpL = named(ggml_add(ctx, inpL, embd_out), "loop_embd", run);
            ggml_tensor * step = ggml_view_1d(ctx, m->loop_step, hp.n_embd, (size_t) m->runs[(size_t) run].pass * m->loop_step->nb[1]);
            inpL = named(ggml_add(ctx, inpL, step), "loop_x", run);
        }
        ggml_tensor * inpSA = inpL;
        ggml_tensor * h = norm_w(ctx, lc, inpL, L.attn_norm, eps, "attn_norm", run);
        ggml_tensor * cur = lc.shift ? build_token_shift(c, ctx, gf, h, L.shift, run, io) : h;
        if (lc.mixer == LLM_MIX_MLSTM) cur = build_mixer_mlstm(c, ctx, gf, L, lc, cur, run, n_tokens, io);
        else if (lc.mixer == LLM_MIX_DELTA) cur = build_mixer_delta(c, ctx, gf, L, lc, cur, run, n_tokens, io);
        else if (lc.mixer == LLM_MIX_SIGMOID_WKV) cur = build_mixer_sigmoid_wkv(c, ctx, gf, L, lc, cur, run, n_tokens, n_kv, io);
        else if (lc.mixer == LLM_MIX_SSD) cur = build_mixer_ssd(c, ctx, gf, L, lc, cur, run, n_tokens, io);
        else if (lc.mixer == LLM_MIX_ATTN_DELTA) cur = build_mixer_attn_delta(c, ctx, gf, L, lc, cur, il, run, n_tokens, n_kv, io);
        else {
            cur = lc.mixer == LLM_MIX_LATENT ? build_mixer_latent(c, ctx, gf, L, lc, cur, il, run, n_tokens, n_kv, io)
                                             : build_mixer_attention(c, ctx, gf, L, lc, cur, il, run, n_tokens, n_kv, io, &v_first);
            cur = named(ggml_mul_mat(ctx, L.wo, cur), "attn_out", run);
        }
        if (lc.parallel) {  // both sublayers read the one normed input (the feed-forward the unshifted one); their sum joins the stream
            if (last && io.out_ids) {  // only the rows whose logits are wanted go on from here
                cur = ggml_get_rows(ctx, cur, io.out_ids);
                inpSA = ggml_get_rows(ctx, inpSA, io.out_ids);
                h = ggml_get_rows(ctx, h, io.out_ids);
            }
            if (lc.two_norms && lc.mlp != LLM_MLP_NONE) h = norm_w(ctx, lc, inpSA, L.ffn_norm, eps, "ffn_norm", run);  // (the feed-forward's own norm of the same x)
            if (lc.mlp != LLM_MLP_NONE) cur = named(ggml_add(ctx, cur, build_ffn(ctx, gf, L, lc, h, il, run)), "mix_ffn", run);
            inpL = named(ggml_add(ctx, inpSA, cur), "l_out", run);
            if (L.side_gate) {
                ggml_tensor * e = named(ggml_get_rows(ctx, L.side_embd, io.tokens), "side_embd", run);
                if (last && io.out_ids) e = ggml_get_rows(ctx, e, io.out_ids);
                ggml_build_forward_expand(gf, e);  // (the rows first: the gate's activation and its product with them then follow one another)
                inpL = build_token_side(ctx, L, inpL, e, eps, run);
            }
            continue;
        }
        if (last && io.out_ids) {
            cur = ggml_get_rows(ctx, cur, io.out_ids);
            inpSA = ggml_get_rows(ctx, inpSA, io.out_ids);
        }
        if (L.attn_post_norm) cur = norm_w(ctx, lc, cur, L.attn_post_norm, eps, "attn_post_norm", run);
        ggml_tensor * ffn_inp = named(ggml_add(ctx, cur, inpSA), lc.mlp == LLM_MLP_NONE ? "l_out" : "ffn_inp", run);
        if (lc.mlp == LLM_MLP_NONE) { inpL = ffn_inp; continue; }
        cur = norm_w(ctx, lc, ffn_inp, L.ffn_norm, eps, "ffn_norm", run);
        cur = build_ffn(ctx, gf, L, lc, cur, il, run);
        if (L.ffn_post_norm) cur = norm_w(ctx, lc, cur, L.ffn_post_norm, eps, "ffn_post_norm", run);
        inpL = named(ggml_add(ctx, cur, ffn_inp), "l_out", run);
    }
    const bool rms_out = !m->lcfg.empty() && m->lcfg[0].rms;
    ggml_tensor * cur = rms_out ? named(ggml_mul(ctx, named(ggml_rms_norm(ctx, inpL, eps), "rnorm", -1), m->output_norm), "result_norm", -1)
                                : layer_norm_w(ctx, inpL, m->output_norm, eps, "result_norm", -1);
    cur = named(ggml_mul_mat(ctx, m->output, cur), m->logit_scale != 1.0f ? "result_unscaled" : "result_output", -1);
    if (m->logit_scale != 1.0f) cur = named(ggml_scale(ctx, cur, m->logit_scale), "result_output", -1);
    ggml_set_output(cur);
    ggml_build_forward_expand(gf, cur);
    io.out = cur;
}

static void build_graph(llm_context * c, int n_tokens, int n_kv, int n_outputs, int n_seqs = 0) {
    if (c->ctx_compute) ggml_free(c->ctx_compute);
    c->ctx_compute = ggml_init({0, nullptr, true});
    ggml_cgraph * gf = ggml_new_graph_custom(c->ctx_compute, 8192, false);
    seg_io io;
    make_inputs(c, c->ctx_compute, 0, c->model->hp.n_layer, true, n_tokens, n_kv, n_outputs, io, n_seqs);
    if (!c->model->lcfg.empty()) build_layerwise(c, c->ctx_compute, gf, n_tokens, n_kv, io);
    else build_segment(c, c->ctx_compute, gf, 0, c->model->hp.n_layer, true, n_tokens, n_kv, io);
    c->inp_masks = io.masks;
    c->inp_tokens = io.tokens;
    c->inp_pos = io.pos;
    c->inp_mask = io.mask;
    c->inp_k_idxs = io.k_idxs;
    c->inp_v_idxs = io.v_idxs;
    c->inp_out_ids = io.out_ids;
    c->inp_bigram = io.bigram_rows;
    c->inp_shift_src = io.shift_src;
    c->inp_shift_last = io.shift_last;
    c->inp_shift_slot = io.shift_slot;
    c->inp_seq_hist = io.seq_hist;
    c->inp_seq_upd = io.seq_upd;
    c->inp_seq_tok = io.seq_tok;
    c->inp_seq_info = io.seq_info;
    c->t_logits = io.out;
    c->gf = gf;
}

extern "C" struct llm_context * llm_context_new(struct llm_model * m, ggml_backend_t backend, llm_compute_fn compute, const struct llm_context_params * p) {
    if ((backend == nullptr) == (compute == nullptr)) {
        fprintf(stderr, "llm_context_new: exactly one of backend / compute must be given\n");
        return nullptr;
    }
    llm_context * c = new llm_context();
    c->model = m;
    c->backend = backend;
    c->compute = compute;
    c->p = *p;
    if (c->p.n_ubatch <= 0) c->p.n_ubatch = 512;
    if (c->p.n_ctx <= 0) c->p.n_ctx = 512;
    c->p.n_ctx = (c->p.n_ctx + 255) / 256 * 256;
    c->buft = backend ? ggml_backend_dev_buffer_type(backend->device) : ggml_backend_cpu_buffer_type();
    const llm_hparams & hp = m->hp;
    const int64_t n_embd_k = (int64_t) m->n_head_kv_l * hp.n_embd_head;
    // -ctk / -ctv (llama-box/engine_param.hpp:51-54): f32, f16, bf16, q8_0, q4_0, q4_1, iq4_nl, q5_0, q5_1.  0 = the default (f16); f32 is ggml type 0
    // too, so it is asked for as LLM_KV_TYPE_F32 (-1)
    auto kv_type_of = [](int32_t t) { return t == 0 ? GGML_TYPE_F16 : t == LLM_KV_TYPE_F32 ? GGML_TYPE_F32 : (ggml_type) t; };
    auto kv_type_ok = [](ggml_type t) {
        return t == GGML_TYPE_F32 || t == GGML_TYPE_F16 || t == GGML_TYPE_BF16 || t == GGML_TYPE_Q8_0 || t == GGML_TYPE_Q4_0 || t == GGML_TYPE_Q4_1 || t == GGML_TYPE_IQ4_NL ||
               t == GGML_TYPE_Q5_0 || t == GGML_TYPE_Q5_1;
    };
    // a model described layer by layer runs its attention as one fused op over a cache kept, by default, in the type of its matrices (bf16 or f32)
    const bool layerwise = !m->lcfg.empty();
    if (layerwise) c->p.flash_attn = 1;
    const ggml_type type_k = (layerwise && c->p.type_k == 0) ? m->wtype : kv_type_of(c->p.type_k), type_v = (layerwise && c->p.type_v == 0) ? m->wtype : kv_type_of(c->p.type_v);
    if (layerwise && (ggml_blck_size(type_k) != 1 || ggml_blck_size(type_v) != 1)) {
        fprintf(stderr, "llm_context_new: a per-layer model keeps its cache in f32, f16 or bf16\n");
        delete c;
        return nullptr;
    }
    // (llama.cpp: a quantised V cache needs flash attention — the non-flash path keeps V transposed, one element per index; K may be of any type there:
    // K.q is then a MUL_MAT over the cache's blocks)
    if (!kv_type_ok(type_k) || !kv_type_ok(type_v) || (type_v != GGML_TYPE_F16 && !c->p.flash_attn) || (hp.n_embd_head % ggml_blck_size(type_k)) != 0 || (hp.n_embd_head % ggml_blck_size(type_v)) != 0) {
        fprintf(stderr, "llm_context_new: unsupported KV cache types %d/%d (f32, f16, bf16, q8_0, q4_0, q4_1, iq4_nl, q5_0, q5_1; a V cache other than f16 needs flash_attn)\n", (int) type_k, (int) type_v);
        delete c;
        return nullptr;
    }
    c->ctx_kv = ggml_init({0, nullptr, true});
    const int n_runs = layerwise ? (int) m->runs.size() : hp.n_layer;
    for (int run = 0; run < n_runs; ++run) {
        // (a model described layer by layer: every layer RUN has a cache of its own, its rows as wide as that layer's keys and values; a latent-attention
        // layer keeps ONE row [latent | rotated key part] per token and no values beside it)
        const llm_layer_cfg * lc = layerwise ? &m->lcfg[(size_t) m->runs[(size_t) run].il] : nullptr;
        const bool latent = lc && lc->mixer == LLM_MIX_LATENT;
        if (lc && (lc->mixer == LLM_MIX_MLSTM || lc->mixer == LLM_MIX_DELTA || lc->mixer == LLM_MIX_SSD || (latent && lc->kv_from >= 0))) {
            // (no cells: everything such a layer keeps is its sequence state — or it attends over the rows another layer's cache holds)
            c->k_l.push_back(nullptr);
            c->v_l.push_back(nullptr);
            continue;
        }
        const int64_t row_k = latent ? (int64_t) lc->kv_rank + lc->rot_dim : lc ? (int64_t) lc->n_head_kv * lc->dk : n_embd_k;
        const int64_t row_v = lc ? (int64_t) lc->n_head_kv * lc->dv : n_embd_k;
        ggml_tensor * k = ggml_new_tensor_2d(c->ctx_kv, type_k, row_k, c->p.n_ctx);
        ggml_tensor * v = latent ? nullptr
                        : c->p.flash_attn ? ggml_new_tensor_2d(c->ctx_kv, type_v, row_v, c->p.n_ctx)
                                          : ggml_new_tensor_2d(c->ctx_kv, GGML_TYPE_F16, c->p.n_ctx, n_embd_k);
        named(k, "cache_k_l", run);
        if (v) named(v, "cache_v_l", run);
        c->k_l.push_back(k);
        c->v_l.push_back(v);
    }
    c->n_seq_max = c->p.n_seq_max > 0 ? c->p.n_seq_max : 8;
    if (m->has_shift || m->bigram || m->has_seq_state) c->seq_prev_tok.assign((size_t) c->n_seq_max, -1);
    if (m->has_seq_state) {
        c->conv_state.assign((size_t) n_runs, nullptr);
        c->tm_shift_state.assign((size_t) n_runs, nullptr);
        c->rec_state.assign((size_t) n_runs, nullptr);
        for (int run = 0; run < n_runs; ++run) {
            const llm_layer_cfg & lc = m->lcfg[(size_t) m->runs[(size_t) run].il];
            const int64_t S = c->n_seq_max;
            int64_t conv_c = 0, rec = 0;
            if (lc.mixer == LLM_MIX_MLSTM) rec = ggml_seq_state_size(2, lc.n_head, lc.dk, lc.dv);
            else if (lc.mixer == LLM_MIX_DELTA) { conv_c = 2 * (int64_t) lc.n_head_kv * lc.dk + (int64_t) lc.n_head * lc.dv; rec = ggml_seq_state_size(1, lc.n_head, lc.dk, lc.dv); }
            else if (lc.mixer == LLM_MIX_SSD) { conv_c = (int64_t) lc.n_head * lc.dv + 2 * (int64_t) lc.ssm_groups * lc.ssm_state; rec = ggml_seq_state_size(4, lc.n_head, lc.ssm_state, lc.dv); }
            else if (lc.mixer == LLM_MIX_ATTN_DELTA) { conv_c = 2 * (int64_t) lc.r_head_kv * lc.r_dk + (int64_t) lc.r_head * lc.r_dv; rec = ggml_seq_state_size(3, lc.r_head, lc.r_dk, lc.r_dv); }
            else if (lc.mixer == LLM_MIX_SIGMOID_WKV) {
                conv_c = (int64_t) (lc.n_head + lc.n_head_kv) * lc.dk + (int64_t) lc.n_head_kv * lc.dv;
                rec = ggml_seq_state_size(0, lc.tm_heads, lc.tm_dim, lc.tm_dim);
                c->tm_shift_state[(size_t) run] = named(ggml_new_tensor_2d(c->ctx_kv, GGML_TYPE_F32, hp.n_embd, S), "time_mix_shift_state", run);
            }
            if (conv_c > 0 && lc.conv_taps > 1) c->conv_state[(size_t) run] = named(ggml_new_tensor_2d(c->ctx_kv, GGML_TYPE_F32, conv_c * (lc.conv_taps - 1), S), "conv_state", run);
            if (rec > 0) c->rec_state[(size_t) run] = named(ggml_new_tensor_2d(c->ctx_kv, GGML_TYPE_F32, rec, S), "recurrence_state", run);
        }
    }
    if (m->has_shift) c->shift_state = named(ggml_new_tensor_3d(c->ctx_kv, GGML_TYPE_F32, hp.n_embd, c->n_seq_max + 1, n_runs), "shift_state", -1);
    c->buf_kv = ggml_backend_alloc_ctx_tensors_from_buft(c->ctx_kv, c->buft);
    if (!c->buf_kv) {
        fprintf(stderr, "llm_context_new: failed to allocate the KV cache\n");
        llm_context_free(c);
        return nullptr;
    }
    ggml_backend_buffer_clear(c->buf_kv, 0);
    c->cells.assign(c->p.n_ctx, kv_cell());
    c->used_max = 0;
    c->galloc = ggml_gallocr_new(c->buft);
    // reserve the worst-case graph (full micro-batch over the full cache) so later graphs re-use one buffer
    build_graph(c, std::min(c->p.n_ubatch, c->p.n_ctx), c->p.n_ctx, std::min(c->p.n_ubatch, c->p.n_ctx),
                (m->has_shift || m->has_seq_state) ? std::min(c->n_seq_max, std::min(c->p.n_ubatch, c->p.n_ctx)) : 0);
    if (!ggml_gallocr_reserve(c->galloc, c->gf)) {
        fprintf(stderr, "llm_context_new: failed to reserve the compute buffer\n");
        llm_context_free(c);
        return nullptr;
    }
    c->key = graph_key();
    if (backend) {
        ggml_backend_buffer_type_t hbuft = ggml_backend_dev_host_buffer_type(backend->device);
        if (hbuft) {
            const size_t nub = (size_t) std::min(c->p.n_ubatch, c->p.n_ctx);
            const size_t n_tok_pad = (nub + 63) / 64 * 64;
            size_t in_bytes = nub * (4 + 4 + 8 + 4) + std::max<size_t>(1, m->mask_rules.size()) * (n_tok_pad * (size_t) c->p.n_ctx * 4 + 64) + 256;
            in_bytes += nub * (4 + 4) + (size_t) c->n_seq_max * (4 + 8) + 4 * 64;  // bigram rows, token-shift sources, the sequences' last rows and state rows
            in_bytes += (nub + (size_t) c->n_seq_max) * (size_t) (m->hist_rows + 4) * 4 + 4 * 64;  // predecessors, new state rows, rows grouped by sequence, the sequences' entries
            if (!c->p.flash_attn) in_bytes += nub * (size_t) n_embd_k * 8;
            in_bytes = (in_bytes + 255) / 256 * 256;
            c->pin_out_rows = 64;
            c->buf_pin = ggml_backend_buft_alloc_buffer(hbuft, in_bytes * llm_context::PIN_SLOTS + (size_t) c->pin_out_rows * m->n_vocab_l * 4);
            if (c->buf_pin) {
                c->pin = (char *) ggml_backend_buffer_get_base(c->buf_pin);
                c->pin_in_bytes = in_bytes;
            }
        }
    }
    return c;
}

extern "C" void llm_context_free(struct llm_context * c) {
    if (!c) return;
    for (auto & d : c->ls) {
        if (d.be) ggml_backend_synchronize(d.be);
        for (int k = 0; k < llm_context::LS_COPIES; ++k) {
            if (d.ctx[k]) ggml_free(d.ctx[k]);
            if (d.ev[k]) ggml_backend_event_free(d.ev[k]);
        }
        if (d.galloc) ggml_gallocr_free(d.galloc);
        if (d.buf_in) ggml_backend_buffer_free(d.buf_in);
        if (d.ctx_in) ggml_free(d.ctx_in);
        if (d.buf_kv) ggml_backend_buffer_free(d.buf_kv);
        if (d.ctx_kv) ggml_free(d.ctx_kv);
    }
    if (c->ctx_compute) ggml_free(c->ctx_compute);
    if (c->galloc) ggml_gallocr_free(c->galloc);
    if (c->buf_pin) ggml_backend_buffer_free(c->buf_pin);
    if (c->buf_kv) ggml_backend_buffer_free(c->buf_kv);
    if (c->ctx_kv) ggml_free(c->ctx_kv);
    delete c;
}

extern "C" void llm_kv_clear(struct llm_context * c) {
    for (auto & x : c->cells) x = kv_cell();
    c->used_max = 0;
    c->kv_head = 0;
}
extern "C" int llm_kv_seq_rm(struct llm_context * c, int seq_id, int p0, int p1) {
    if (p0 < 0) p0 = 0;
    if (p1 < 0) p1 = INT32_MAX;
    for (auto & x : c->cells)
        if (x.pos >= p0 && x.pos < p1 && (seq_id < 0 || x.seq == seq_id)) { x = kv_cell(); c->used_max = -1; }
    c->kv_head = 0;
    return 1;
}

// K-shift: the graph llama.cpp's llama_kv_cache::build_rope_shift produces after llama_memory_seq_add (llama-box context
// shift, httpserver.hpp:3453-3537).  Every cell's K row is rotated by the cell's position delta: in place on an f16 cache;
// on a quantised cache through an f32 copy (cast -> rope -> cpy back, which re-quantises the rows).
static int kv_apply_shift(llm_context * c, const std::vector<int32_t> & delta) {
    llm_model * m = c->model;
    const llm_hparams & hp = m->hp;
    const int64_t HD = hp.n_embd_head, NKV = m->n_head_kv_l, n_ctx = c->p.n_ctx;
    if (c->backend && c->in_flight) { ggml_backend_synchronize(c->backend); c->in_flight = 0; }
    ggml_context * ctx = ggml_init({0, nullptr, true});
    ggml_cgraph * gf = ggml_new_graph_custom(ctx, 1024, false);
    ggml_tensor * shift = ggml_new_tensor_1d(ctx, GGML_TYPE_I32, n_ctx);
    ggml_set_input(named(shift, "k_shift", -1));
    for (int il = 0; il < hp.n_layer; ++il) {
        ggml_tensor * kc = c->k_l[il];
        ggml_tensor * k = ggml_view_3d(ctx, kc, HD, NKV, n_ctx, ggml_row_size(kc->type, HD), ggml_row_size(kc->type, NKV * HD), 0);
        ggml_tensor * r;
        if (kc->type == GGML_TYPE_BF16) {  // (llama.cpp ropes a non-quantised cache in place, and ROPE has no bf16 form: no context shift on such a cache)
            ggml_free(ctx);
            return -2;
        }
        if (ggml_blck_size(kc->type) > 1) {  // ggml_is_quantized
            ggml_tensor * tmp = ggml_cast(ctx, k, GGML_TYPE_F32);
            tmp = ggml_rope_ext_inplace(ctx, tmp, shift, nullptr, (int) HD, hp.rope_type, hp.n_ctx_train, hp.rope_freq_base, 1.0f, 0.0f, 1.0f, 32.0f, 1.0f);
            r = ggml_cpy(ctx, tmp, k);
        } else {
            r = ggml_rope_ext_inplace(ctx, k, shift, nullptr, (int) HD, hp.rope_type, hp.n_ctx_train, hp.rope_freq_base, 1.0f, 0.0f, 1.0f, 32.0f, 1.0f);
        }
        ggml_build_forward_expand(gf, named(r, "k_shifted", il));
    }
    ggml_gallocr_t ga = ggml_gallocr_new(c->buft);
    int rc = 0;
    if (!ga || !ggml_gallocr_alloc_graph(ga, gf)) rc = -2;
    if (rc == 0) {
        ggml_backend_tensor_set(shift, delta.data(), 0, (size_t) n_ctx * 4);
        const enum ggml_status st = c->backend ? ggml_backend_graph_compute(c->backend, gf) : c->compute(gf, c->p.n_threads);
        if (st != GGML_STATUS_SUCCESS) rc = -2;
    }
    if (ga) ggml_gallocr_free(ga);
    ggml_free(ctx);
    return rc;
}
// llama_memory_seq_add: positions [p0, p1) of a sequence move by `delta`; the cached K rows are re-rotated at once
// (llama.cpp defers that to the next llama_decode's memory update — same result).  Returns 0, or -2 if the shift graph failed.
extern "C" int llm_kv_seq_add(struct llm_context * c, int seq_id, int p0, int p1, int delta) {
    if (!c->ls.empty()) return -2;  // (the K-shift graph is not cut over devices in this harness)
    if (c->model->has_shift) return -2;  // (sequence state beside the cache: positions of such a model do not move)
    if (p0 < 0) p0 = 0;
    if (p1 < 0) p1 = INT32_MAX;
    if (delta == 0) return 0;
    std::vector<int32_t> d((size_t) c->p.n_ctx, 0);
    bool any = false;
    for (size_t i = 0; i < c->cells.size(); ++i) {
        kv_cell & x = c->cells[i];
        if (x.pos >= p0 && x.pos < p1 && (seq_id < 0 || x.seq == seq_id)) {
            x.pos += delta;
            d[i] = delta;
            any = true;
            if (x.pos < 0) { x = kv_cell(); c->used_max = -1; }  // shifted out of the sequence (llama.cpp frees such cells too)
        }
    }
    return any ? kv_apply_shift(c, d) : 0;
}

// ------------------------------------------------------------------------------------------------ -sm layer
// llama.cpp's default with several devices (llama-box/engine_param.hpp:900-916: split_mode stays LLAMA_SPLIT_MODE_LAYER unless -sm says
// otherwise; patches/llama.cpp/max_devices.patch:5-10 raises the device limit): every device holds a range of layers and their KV cache,
// ggml_backend_sched cuts the graph where the weights change device and moves the residual stream across with the destination backend's
// cpy_tensor_async, ordering the re-use of its input copies with event_record / event_wait / event_synchronize.  This is that driver for
// OUR devices (no scheduler exists in the snapshot): the calls a backend sees, in the order ggml_backend_sched_compute_splits issues them.
extern "C" struct llm_context * llm_context_new_layer_split(struct llm_model * m, const ggml_backend_t * backends, int n_dev, const struct llm_context_params * p) {
    if (n_dev < 1 || n_dev != m->n_dev || (int) m->layer_dev.size() != m->hp.n_layer) {
        fprintf(stderr, "llm_context_new_layer_split: the model was not built by llm_model_synth_layer_split for %d devices\n", n_dev);
        return nullptr;
    }
    llm_context * c = new llm_context();
    c->model = m;
    c->p = *p;
    if (c->p.n_ubatch <= 0) c->p.n_ubatch = 512;
    if (c->p.n_ctx <= 0) c->p.n_ctx = 512;
    c->p.n_ctx = (c->p.n_ctx + 255) / 256 * 256;
    const llm_hparams & hp = m->hp;
    const int64_t n_embd_k = (int64_t) m->n_head_kv_l * hp.n_embd_head;
    c->ls.resize((size_t) n_dev);
    c->k_l.assign((size_t) hp.n_layer, nullptr);
    c->v_l.assign((size_t) hp.n_layer, nullptr);
    for (int d = 0; d < n_dev; ++d) {
        llm_context::ls_dev & D = c->ls[(size_t) d];
        D.be = backends[d];
        D.buft = ggml_backend_dev_buffer_type(backends[d]->device);
        D.l0 = hp.n_layer;
        D.l1 = 0;
        for (int il = 0; il < hp.n_layer; ++il)
            if (m->layer_dev[(size_t) il] == d) { D.l0 = std::min(D.l0, il); D.l1 = std::max(D.l1, il + 1); }
        LLM_ASSERT(D.l0 < D.l1);
        D.ctx_kv = ggml_init({0, nullptr, true});
        for (int il = D.l0; il < D.l1; ++il) {
            ggml_tensor * k = ggml_new_tensor_2d(D.ctx_kv, GGML_TYPE_F16, n_embd_k, c->p.n_ctx);
            ggml_tensor * v = c->p.flash_attn ? ggml_new_tensor_2d(D.ctx_kv, GGML_TYPE_F16, n_embd_k, c->p.n_ctx) : ggml_new_tensor_2d(D.ctx_kv, GGML_TYPE_F16, c->p.n_ctx, n_embd_k);
            c->k_l[(size_t) il] = named(k, "cache_k_l", il);
            c->v_l[(size_t) il] = named(v, "cache_v_l", il);
        }
        D.buf_kv = ggml_backend_alloc_ctx_tensors_from_buft(D.ctx_kv, D.buft);
        if (!D.buf_kv) { llm_context_free(c); return nullptr; }
        ggml_backend_buffer_clear(D.buf_kv, 0);
        D.galloc = ggml_gallocr_new(D.buft);
        for (int k = 0; k < llm_context::LS_COPIES; ++k) D.ev[k] = ggml_backend_event_new(backends[d]->device);
        // reserve the worst-case segment so that later graphs re-use one buffer
        const int nub = std::min(c->p.n_ubatch, c->p.n_ctx);
        ggml_context * tmp = ggml_init({0, nullptr, true});
        ggml_cgraph * gf = ggml_new_graph_custom(tmp, 8192, false);
        seg_io io;
        make_inputs(c, tmp, D.l0, D.l1, d == n_dev - 1, nub, c->p.n_ctx, nub, io);
        build_segment(c, tmp, gf, D.l0, D.l1, d == n_dev - 1, nub, c->p.n_ctx, io);
        const bool ok = ggml_gallocr_reserve(D.galloc, gf);
        ggml_free(tmp);
        if (!ok) { llm_context_free(c); return nullptr; }
    }
    c->cells.assign((size_t) c->p.n_ctx, kv_cell());
    c->used_max = 0;
    c->key = graph_key();
    return c;
}
extern "C" void llm_layer_split_stats(const struct llm_context * c, int64_t out[4]) {
    for (int k = 0; k < 4; ++k) out[k] = c->ls_stats[k];
}

static void ls_sync_all(llm_context * c) {
    for (auto & d : c->ls) ggml_backend_synchronize(d.be);
    c->ls_copy = 0;  // ggml_backend_sched_synchronize: "always use copy 0 after a synchronization" — a decode step sees the same graph every time
    c->in_flight = 0;
}

static int decode_ubatch_ls(llm_context * c, int n_tokens, const int32_t * tokens, const int32_t * pos, const int32_t * seq_id, const std::vector<int> & slots,
                            const std::vector<int32_t> & out_ids, int n_kv, float * logits_out, int * n_out_acc, bool defer_sync) {
    llm_model * m = c->model;
    const llm_hparams & hp = m->hp;
    const int n_ctx = c->p.n_ctx, n_dev = (int) c->ls.size(), n_outputs = (int) out_ids.size();
    const int64_t n_embd_k = (int64_t) m->n_head_kv_l * hp.n_embd_head;
    graph_key key{n_tokens, n_kv, n_outputs};
    if (!(key == c->key)) {
        ls_sync_all(c);
        for (int d = 0; d < n_dev; ++d) {
            llm_context::ls_dev & D = c->ls[(size_t) d];
            if (D.buf_in) ggml_backend_buffer_free(D.buf_in);
            if (D.ctx_in) ggml_free(D.ctx_in);
            D.ctx_in = ggml_init({0, nullptr, true});
            for (int k = 0; k < llm_context::LS_COPIES; ++k) {
                D.io[k] = seg_io();
                make_inputs(c, D.ctx_in, D.l0, D.l1, d == n_dev - 1, n_tokens, n_kv, n_outputs, D.io[k]);
            }
            D.buf_in = ggml_backend_alloc_ctx_tensors_from_buft(D.ctx_in, D.buft);
            if (!D.buf_in) return -2;
            for (int k = 0; k < llm_context::LS_COPIES; ++k) {
                if (D.ctx[k]) ggml_free(D.ctx[k]);
                D.ctx[k] = ggml_init({0, nullptr, true});
                D.gf[k] = ggml_new_graph_custom(D.ctx[k], 8192, false);
                build_segment(c, D.ctx[k], D.gf[k], D.l0, D.l1, d == n_dev - 1, n_tokens, n_kv, D.io[k]);
                if (!ggml_gallocr_alloc_graph(D.galloc, D.gf[k])) return -2;  // (same topology, same plan: both slots' graphs share the compute buffer — they run one after the other on the device's stream)
            }
            // the padding rows of the masks (GGML_KQ_MASK_PAD) are never read; written once so that the cast never converts uninitialised memory
            for (int k = 0; k < llm_context::LS_COPIES; ++k) {
                std::vector<float> pad((size_t) D.io[k].mask->ne[0] * (size_t) D.io[k].mask->ne[1], -INFINITY);
                ggml_backend_tensor_set(D.io[k].mask, pad.data(), 0, pad.size() * 4);
            }
        }
        c->key = key;
    }
    const int cur = c->ls_copy;
    // host-side images of the user inputs
    std::vector<int64_t> kidx((size_t) n_tokens), vidx;
    for (int i = 0; i < n_tokens; ++i) kidx[(size_t) i] = slots[(size_t) i];
    if (!c->p.flash_attn) {
        vidx.resize((size_t) n_tokens * (size_t) n_embd_k);
        for (int i = 0; i < n_tokens; ++i)
            for (int64_t j = 0; j < n_embd_k; ++j) vidx[(size_t) i * n_embd_k + j] = j * n_ctx + slots[(size_t) i];
    }
    std::vector<int32_t> & cpos = c->mask_cpos, & cseq = c->mask_cseq;
    cpos.resize((size_t) n_kv);
    cseq.resize((size_t) n_kv);
    for (int j = 0; j < n_kv; ++j) { cpos[(size_t) j] = c->cells[(size_t) j].pos; cseq[(size_t) j] = c->cells[(size_t) j].seq; }
    std::vector<float> mask((size_t) n_kv * (size_t) n_tokens);
    for (int i = 0; i < n_tokens; ++i) mask_row(mask.data() + (size_t) i * n_kv, n_kv, cpos.data(), cseq.data(), seq_id ? seq_id[i] : 0, pos[i], 0.0f, -INFINITY);

    enum ggml_status st = GGML_STATUS_SUCCESS;
    for (int d = 0; d < n_dev && st == GGML_STATUS_SUCCESS; ++d) {
        llm_context::ls_dev & D = c->ls[(size_t) d];
        seg_io & io = D.io[cur];
        // --- user inputs (GGML_TENSOR_FLAG_INPUT): the split backend must have finished the graph that read this slot last, then a BLOCKING copy
        if (D.ev[cur]) ggml_backend_event_synchronize(D.ev[cur]);
        else ggml_backend_synchronize(D.be);
        if (d == 0) {
            // (llama.cpp fills its input tensors with ggml_backend_tensor_set — blocking — from host memory)
            if (io.tokens) ggml_backend_tensor_set(io.tokens, tokens, 0, (size_t) n_tokens * 4);
            ggml_backend_tensor_set(io.pos, pos, 0, (size_t) n_tokens * 4);
            ggml_backend_tensor_set(io.k_idxs, kidx.data(), 0, kidx.size() * 8);
            if (io.v_idxs) ggml_backend_tensor_set(io.v_idxs, vidx.data(), 0, vidx.size() * 8);
            ggml_backend_tensor_set(io.mask, mask.data(), 0, mask.size() * 4);
            if (io.out_ids) ggml_backend_tensor_set(io.out_ids, out_ids.data(), 0, out_ids.size() * 4);
        } else {
            // an input that lives on another device's backend: ggml_backend_tensor_copy -> the destination buffer's cpy_tensor
            seg_io & src = c->ls[0].io[cur];
            ggml_backend_tensor_copy(src.pos, io.pos);
            ggml_backend_tensor_copy(src.k_idxs, io.k_idxs);
            if (io.v_idxs) ggml_backend_tensor_copy(src.v_idxs, io.v_idxs);
            ggml_backend_tensor_copy(src.mask, io.mask);
            c->ls_stats[1] += 3 + (io.v_idxs ? 1 : 0);
            if (io.out_ids) ggml_backend_tensor_set(io.out_ids, out_ids.data(), 0, out_ids.size() * 4);  // (only the last device reads it: its own input)
            // --- the residual stream, produced by the previous device's graph: wait until this backend is done with the slot, then the async copy
            llm_context::ls_dev & P = c->ls[(size_t) d - 1];
            if (D.ev[cur]) { ggml_backend_event_wait(D.be, D.ev[cur]); c->ls_stats[3]++; }
            else ggml_backend_synchronize(D.be);
            // (harness addition, not in ggml_backend_sched: the copy is issued on the SOURCE stream — also order it behind the destination's last use of the slot)
            if (D.ev[cur]) { ggml_backend_event_wait(P.be, D.ev[cur]); c->ls_stats[3]++; }
            ggml_backend_tensor_copy_async(P.be, D.be, P.io[cur].out, io.resid);
            c->ls_stats[0]++;
        }
        st = ggml_backend_graph_compute_async(D.be, D.gf[cur]);
        if (D.ev[cur]) { ggml_backend_event_record(D.ev[cur], D.be); c->ls_stats[2]++; }
    }
    if (st != GGML_STATUS_SUCCESS) { ls_sync_all(c); return -2; }
    if (n_outputs > 0 || !defer_sync) {
        llm_context::ls_dev & Last = c->ls.back();
        if (n_outputs > 0) ggml_backend_tensor_get_async(Last.be, Last.io[cur].out, logits_out, 0, (size_t) n_outputs * m->n_vocab_l * 4);
        ls_sync_all(c);
        *n_out_acc += n_outputs;
        c->t_logits = Last.io[cur].out;
        c->gf = Last.gf[cur];
    } else {
        c->ls_copy = (cur + 1) % llm_context::LS_COPIES;  // the next micro-batch takes the other slot while this one is in flight
        c->in_flight++;
    }
    return 0;
}

static int decode_ubatch(llm_context * c, int n_tokens, const int32_t * tokens, const int32_t * pos, const int32_t * seq_id, const int8_t * want, float * logits_out, int * n_out_acc,
                         bool defer_sync) {
    llm_model * m = c->model;
    const llm_hparams & hp = m->hp;
    const int n_ctx = c->p.n_ctx;
    const double t0 = now_us();
    // find free cells (first fit from kv_head, wrapping once)
    std::vector<int> slots;
    for (int i = 0, at = c->kv_head; i < n_ctx && (int) slots.size() < n_tokens; ++i, at = (at + 1) % n_ctx)
        if (c->cells[at].pos < 0) slots.push_back(at);
    if ((int) slots.size() < n_tokens) return 1;
    for (int i = 0; i < n_tokens; ++i) {
        c->cells[slots[i]].pos = pos[i];
        c->cells[slots[i]].seq = seq_id ? seq_id[i] : 0;
    }
    c->kv_head = (slots.back() + 1) % n_ctx;
    // (kept up to date by the allocations; a full recount only after cells were freed)
    if (c->used_max < 0) {
        c->used_max = 0;
        for (int i = 0; i < n_ctx; ++i) if (c->cells[i].pos >= 0) c->used_max = i + 1;
    }
    for (int i = 0; i < n_tokens; ++i) c->used_max = std::max(c->used_max, slots[i] + 1);
    const int used_max = c->used_max;
    const int n_kv = std::min(n_ctx, (used_max + 255) / 256 * 256);
    std::vector<int32_t> out_ids;
    for (int i = 0; i < n_tokens; ++i) if (!want || want[i]) out_ids.push_back(i);
    const int n_outputs = (int) out_ids.size();
    // a micro-batch nobody wants logits from (every chunk of a prompt but the last): llama.cpp builds the graph with an EMPTY out_ids — the last
    // layer's tensors behind get_rows and the output head have zero rows and are skipped by the backends (ggml_is_empty)
    const int n_out_graph = n_outputs;
    if (!c->ls.empty()) {
        const int rc = decode_ubatch_ls(c, n_tokens, tokens, pos, seq_id, slots, out_ids, n_kv, logits_out, n_out_acc, defer_sync);
        if (rc != 0) {
            for (int i = 0; i < n_tokens; ++i) c->cells[slots[i]] = kv_cell();
            c->used_max = -1;
        }
        return rc;
    }

    // sequence state (models with a hashed bigram embedding / token shift): where every token finds its predecessor — the row before it in this
    // micro-batch, or its sequence's state — and which token of each sequence is the last one here.  A token at position 0 has no predecessor
    std::vector<int32_t> bigram_rows, shift_src, shift_last;
    std::vector<int64_t> shift_slot;
    std::vector<int32_t> new_prev_tok;
    if (m->has_shift || m->bigram) {
        const int S = c->n_seq_max;
        std::vector<int> last_in_batch((size_t) S, -1);
        new_prev_tok = c->seq_prev_tok;
        bigram_rows.resize((size_t) n_tokens);
        shift_src.resize((size_t) n_tokens);
        for (int i = 0; i < n_tokens; ++i) {
            const int sq = seq_id ? seq_id[i] : 0;
            const int before = last_in_batch[(size_t) sq];
            const bool first = pos[i] == 0;
            const int32_t prev_tok = before >= 0 ? tokens[before] : new_prev_tok[(size_t) sq];
            if (first || prev_tok < 0) bigram_rows[(size_t) i] = m->bg_buckets;
            else bigram_rows[(size_t) i] = (int32_t) (((int64_t) prev_tok * m->bg_mul_prev + (int64_t) tokens[i] * m->bg_mul_cur) % m->bg_buckets);
            shift_src[(size_t) i] = first ? n_tokens + S : before >= 0 ? before : n_tokens + sq;  // rows of [h of the batch | state rows | zero row]
            last_in_batch[(size_t) sq] = i;
        }
        for (int sq = 0; sq < S; ++sq)
            if (last_in_batch[(size_t) sq] >= 0) {
                shift_last.push_back(last_in_batch[(size_t) sq]);
                shift_slot.push_back(sq);
                new_prev_tok[(size_t) sq] = tokens[last_in_batch[(size_t) sq]];
            }
    }
    // layers with convolution / recurrence state: the batch rows of every sequence in their order, and from them where each token's predecessors are found (hist),
    // where the state rows after the batch come from (upd), and the sequences' entries (info)
    std::vector<int32_t> seq_hist, seq_upd, seq_tok, seq_info;
    if (m->has_seq_state) {
        const int S = c->n_seq_max, hs = m->hist_rows;
        std::vector<std::vector<int>> rows((size_t) S);
        for (int i = 0; i < n_tokens; ++i) rows[(size_t) (seq_id ? seq_id[i] : 0)].push_back(i);
        seq_hist.assign((size_t) hs * n_tokens, -1);
        for (int sq = 0; sq < S; ++sq) {
            const std::vector<int> & r = rows[(size_t) sq];
            if (r.empty()) continue;
            const int n = (int) r.size();
            for (int k = 0; k < n; ++k)
                for (int d = 1; d <= hs; ++d) {
                    int32_t code = -1;  // before the sequence's start
                    if (pos[r[(size_t) k]] - d >= 0) code = d <= k ? r[(size_t) (k - d)] : -2 - (sq * 64 + (d - 1 - k));
                    seq_hist[(size_t) r[(size_t) k] * hs + (d - 1)] = code;
                }
            const int last_pos = pos[r[(size_t) (n - 1)]];
            for (int a = 0; a < hs; ++a) {
                int32_t code = -1;
                if (last_pos - a >= 0) code = a < n ? r[(size_t) (n - 1 - a)] : -2 - (sq * 64 + (a - n));
                seq_upd.push_back(code);
            }
            seq_info.push_back((int32_t) seq_tok.size());
            seq_info.push_back(n);
            seq_info.push_back(sq);
            seq_info.push_back(pos[r[0]] == 0 ? 1 : 0);
            for (int k = 0; k < n; ++k) seq_tok.push_back(r[(size_t) k]);
        }
    }
    const int n_seqs = m->has_shift ? (int) shift_last.size() : m->has_seq_state ? (int) (seq_info.size() / 4) : 0;
    graph_key key{n_tokens, n_kv, n_out_graph, n_seqs};
    bool rebuilt = false;
    if (!(c->p.graph_reuse && key == c->key && c->gf)) {
        rebuilt = true;
        build_graph(c, n_tokens, n_kv, n_out_graph, n_seqs);
        if (!ggml_gallocr_alloc_graph(c->galloc, c->gf)) return -2;
        c->key = key;
    }
    const double t1 = now_us();

    // inputs: filled straight into the pinned staging area and uploaded asynchronously on the backend's stream (the copies
    // and the graph are stream-ordered); without a device backend (CPU oracle) the plain blocking setter is used
    const bool async_io = c->backend != nullptr && c->pin != nullptr;
    if (async_io && c->in_flight >= llm_context::PIN_SLOTS - 1) {  // the slot about to be re-used may still be in flight
        ggml_backend_synchronize(c->backend);
        c->in_flight = 0;
    }
    char * const pin_in = c->pin ? c->pin + (size_t) c->pin_slot * c->pin_in_bytes : nullptr;
    char * const pin_out = c->pin ? c->pin + (size_t) llm_context::PIN_SLOTS * c->pin_in_bytes : nullptr;
    c->pin_slot = (c->pin_slot + 1) % llm_context::PIN_SLOTS;
    size_t pin_at = 0;
    std::vector<char> heap;  // CPU-oracle path
    auto upload = [&](ggml_tensor * t, size_t bytes, auto fill) {
        char * dst;
        if (async_io) {
            pin_at = (pin_at + 63) / 64 * 64;
            LLM_ASSERT(pin_at + bytes <= c->pin_in_bytes);
            dst = pin_in + pin_at;
            pin_at += bytes;
        } else {
            heap.resize(bytes);
            dst = heap.data();
        }
        fill(dst);
        if (async_io) ggml_backend_tensor_set_async(c->backend, t, dst, 0, bytes);
        else ggml_backend_tensor_set(t, dst, 0, bytes);
    };
    upload(c->inp_tokens, (size_t) n_tokens * 4, [&](char * d) { memcpy(d, tokens, (size_t) n_tokens * 4); });
    if (c->inp_pos) upload(c->inp_pos, (size_t) n_tokens * 4, [&](char * d) { memcpy(d, pos, (size_t) n_tokens * 4); });
    if (c->inp_k_idxs) upload(c->inp_k_idxs, (size_t) n_tokens * 8, [&](char * d) {
        int64_t * k = (int64_t *) d;
        for (int i = 0; i < n_tokens; ++i) k[i] = slots[i];
    });
    if (c->inp_seq_hist) {
        upload(c->inp_seq_hist, seq_hist.size() * 4, [&](char * d) { memcpy(d, seq_hist.data(), seq_hist.size() * 4); });
        upload(c->inp_seq_upd, seq_upd.size() * 4, [&](char * d) { memcpy(d, seq_upd.data(), seq_upd.size() * 4); });
    }
    if (c->inp_seq_tok) {
        upload(c->inp_seq_tok, seq_tok.size() * 4, [&](char * d) { memcpy(d, seq_tok.data(), seq_tok.size() * 4); });
        upload(c->inp_seq_info, seq_info.size() * 4, [&](char * d) { memcpy(d, seq_info.data(), seq_info.size() * 4); });
    }
    if (c->inp_v_idxs) {
        const int64_t n_embd_k = (int64_t) m->n_head_kv_l * hp.n_embd_head;
        upload(c->inp_v_idxs, (size_t) n_tokens * n_embd_k * 8, [&](char * d) {
            int64_t * vidx = (int64_t *) d;
            for (int i = 0; i < n_tokens; ++i)
                for (int64_t j = 0; j < n_embd_k; ++j) vidx[(size_t) i * n_embd_k + j] = j * n_ctx + slots[i];
        });
    }
    if (c->inp_out_ids) upload(c->inp_out_ids, (size_t) n_out_graph * 4, [&](char * d) { memcpy(d, out_ids.data(), (size_t) n_out_graph * 4); });
    if (c->inp_bigram) upload(c->inp_bigram, (size_t) n_tokens * 4, [&](char * d) { memcpy(d, bigram_rows.data(), (size_t) n_tokens * 4); });
    if (c->inp_shift_src) {
        upload(c->inp_shift_src, (size_t) n_tokens * 4, [&](char * d) { memcpy(d, shift_src.data(), (size_t) n_tokens * 4); });
        upload(c->inp_shift_last, (size_t) n_seqs * 4, [&](char * d) { memcpy(d, shift_last.data(), (size_t) n_seqs * 4); });
        upload(c->inp_shift_slot, (size_t) n_seqs * 8, [&](char * d) { memcpy(d, shift_slot.data(), (size_t) n_seqs * 8); });
    }
    if (c->inp_mask) {
        // rows beyond n_tokens are padding (GGML_KQ_MASK_PAD) that no kernel reads: they are written once when the
        // graph is (re)built and skipped on re-use, which keeps the per-step upload at n_tokens * n_kv entries
        const int64_t n_tok_pad = c->inp_mask->ne[1];
        const int64_t rows = rebuilt ? n_tok_pad : n_tokens;
        // cell j is visible to token i iff it holds a position (>= 0) of i's sequence that is not after i's — the condition llama.cpp's
        // set_input_kq_mask evaluates per (token, cell); the cells' fields are gathered once per step so that the row loops vectorise
        // (an empty cell's position -1 compares as the largest unsigned value: never visible)
        std::vector<int32_t> & cpos = c->mask_cpos, & cseq = c->mask_cseq;
        cpos.resize((size_t) n_kv);
        cseq.resize((size_t) n_kv);
        for (int j = 0; j < n_kv; ++j) {
            cpos[j] = c->cells[j].pos;
            cseq[j] = c->cells[j].seq;
        }
        for (size_t mk = 0; mk < c->inp_masks.size(); ++mk) {
            const llm_mask_rule rule = mk < m->mask_rules.size() ? m->mask_rules[mk] : llm_mask_rule();
            const int chunk = rule.chunk;
            upload(c->inp_masks[mk], (size_t) n_kv * rows * 4, [&](char * d) {
                float * mask = (float *) d;
                for (size_t e = (size_t) n_kv * n_tokens; e < (size_t) n_kv * rows; ++e) mask[e] = -INFINITY;
                for (int i = 0; i < n_tokens; ++i) {
                    if (rule.window > 0 || rule.distance)
                        mask_row_window(mask + (size_t) i * n_kv, n_kv, cpos.data(), cseq.data(), seq_id ? seq_id[i] : 0, pos[i], rule.window, rule.keep_first, rule.distance, -INFINITY);
                    else if (chunk > 0) mask_row_chunked(mask + (size_t) i * n_kv, n_kv, cpos.data(), cseq.data(), seq_id ? seq_id[i] : 0, pos[i], chunk, 0.0f, -INFINITY);
                    else mask_row(mask + (size_t) i * n_kv, n_kv, cpos.data(), cseq.data(), seq_id ? seq_id[i] : 0, pos[i], 0.0f, -INFINITY);
                }
            });
        }
    }
    const double t2 = now_us();
    const size_t logit_bytes = (size_t) n_outputs * m->n_vocab_l * 4;
    // (logits_out inside the pinned output area: llm_decode found room for ALL outputs of the call there — the device writes the
    // rows where llm_get_logits will read them, as llama.cpp's pinned output buffer works; otherwise staged + copied)
    const bool direct_out = c->pin != nullptr && (char *) logits_out >= pin_out && (char *) logits_out < pin_out + (size_t) c->pin_out_rows * m->n_vocab_l * 4;
    const bool async_out = async_io && n_outputs > 0 && (direct_out || n_outputs <= c->pin_out_rows);
    enum ggml_status st;
    if (async_io) {
        st = ggml_backend_graph_compute_async(c->backend, c->gf);
        if (st == GGML_STATUS_SUCCESS && async_out) ggml_backend_tensor_get_async(c->backend, c->t_logits, direct_out ? (void *) logits_out : (void *) pin_out, 0, logit_bytes);
        if (n_outputs > 0 || st != GGML_STATUS_SUCCESS || !defer_sync) {
            ggml_backend_synchronize(c->backend);
            c->in_flight = 0;
        } else {
            c->in_flight++;
        }
    } else {
        st = c->backend ? ggml_backend_graph_compute(c->backend, c->gf) : c->compute(c->gf, c->p.n_threads);
    }
    const double t3 = now_us();
    if (st != GGML_STATUS_SUCCESS) {
        for (int i = 0; i < n_tokens; ++i) c->cells[slots[i]] = kv_cell();  // roll the slots back
        c->used_max = -1;
        return -2;
    }
    if (n_outputs > 0) {
        if (async_out && !direct_out) memcpy(logits_out, pin_out, logit_bytes);
        else if (!async_out) ggml_backend_tensor_get(c->t_logits, logits_out, 0, logit_bytes);
        *n_out_acc += n_outputs;
    }
    if (!new_prev_tok.empty()) c->seq_prev_tok.swap(new_prev_tok);
    const double t4 = now_us();
    c->timings[0] += t1 - t0;
    c->timings[1] += t2 - t1;
    c->timings[2] += t3 - t2;
    c->timings[3] += t4 - t3;
    return 0;
}

extern "C" int llm_decode(struct llm_context * c, int n_tokens, const int32_t * tokens, const int32_t * pos, const int32_t * seq_id, const int8_t * want_logits) {
    if (n_tokens <= 0 || !tokens || !pos) return -1;
    for (int i = 0; i < n_tokens; ++i)
        if (tokens[i] < 0 || tokens[i] >= c->model->hp.n_vocab || pos[i] < 0) return -1;
    if (!c->seq_prev_tok.empty())  // a model with state per sequence: the ids index its state rows
        for (int i = 0; i < n_tokens; ++i)
            if (seq_id && (seq_id[i] < 0 || seq_id[i] >= c->n_seq_max)) return -1;
    int n_total_out = 0;
    for (int i = 0; i < n_tokens; ++i) n_total_out += (!want_logits || want_logits[i]) ? 1 : 0;
    // outputs land in the pinned area when they all fit (one sampled row per sequence: always, up to 64 sequences)
    const bool pinned_out = c->backend != nullptr && c->pin != nullptr && n_total_out <= c->pin_out_rows;
    if (pinned_out) {
        c->logits_base = (float *) (c->pin + (size_t) llm_context::PIN_SLOTS * c->pin_in_bytes);
    } else {
        c->logits.resize((size_t) std::max(1, n_total_out) * c->model->n_vocab_l);
        c->logits_base = c->logits.data();
    }
    c->n_outputs = 0;
    // batch position -> output row (llama.cpp's output_ids): what llama_get_logits_ith(ctx, i) resolves i >= 0 through
    c->output_ids.assign((size_t) n_tokens, -1);
    for (int i = 0, o = 0; i < n_tokens; ++i) if (!want_logits || want_logits[i]) c->output_ids[(size_t) i] = o++;
    for (int k = 0; k < 4; ++k) c->timings[k] = 0;
    for (int i0 = 0; i0 < n_tokens; i0 += c->p.n_ubatch) {
        const int n = std::min(c->p.n_ubatch, n_tokens - i0);
        int rc = decode_ubatch(c, n, tokens + i0, pos + i0, seq_id ? seq_id + i0 : nullptr, want_logits ? want_logits + i0 : nullptr,
                               c->logits_base + (size_t) c->n_outputs * c->model->n_vocab_l, &c->n_outputs, /*defer_sync=*/i0 + n < n_tokens);
        if (rc != 0) {
            if (c->backend && c->in_flight) { ggml_backend_synchronize(c->backend); c->in_flight = 0; }
            if (!c->ls.empty()) ls_sync_all(c);
            return rc;
        }
    }
    if (!c->ls.empty() && c->in_flight) ls_sync_all(c);
    if (c->backend && c->in_flight) {  // the call returns with everything finished
        ggml_backend_synchronize(c->backend);
        c->in_flight = 0;
    }
    return 0;
}
extern "C" int llm_decode_steps(struct llm_context * c, int n_steps, int n_par, const int32_t * tokens, int pos0) {
    if (n_steps <= 0 || n_par <= 0 || !tokens) return -1;
    std::vector<int32_t> pos((size_t) n_par), seq((size_t) n_par);
    for (int s = 0; s < n_par; ++s) seq[s] = s;
    double acc[4] = {0, 0, 0, 0};
    for (int i = 0; i < n_steps; ++i) {
        for (int s = 0; s < n_par; ++s) pos[s] = pos0 + i;
        const int rc = llm_decode(c, n_par, tokens + (size_t) i * n_par, pos.data(), seq.data(), nullptr);
        if (rc != 0) return rc;
        for (int k = 0; k < 4; ++k) acc[k] += c->timings[k];
    }
    for (int k = 0; k < 4; ++k) c->timings[k] = acc[k];
    return 0;
}
// Speculative decoding as llama-box drives it (httpserver.hpp:4042-4069: every slot's sampled token plus its drafts go into ONE batch, logits
// requested at every position; :4696-4768: the drafts are verified against them and the rejected tail is removed from the cache with
// llama_memory_seq_rm).  One step here = one llama_decode over n_par x (1 + n_draft) tokens — sequence s at positions p .. p + n_draft —
// followed by the WORST case of the verification: every draft rejected (seq_rm of p + 1 ..), so the next step starts at p + 1.
// tokens: [n_steps][n_par][1 + n_draft].
extern "C" int llm_verify_steps(struct llm_context * c, int n_steps, int n_par, int n_draft, const int32_t * tokens, int pos0) {
    if (n_steps <= 0 || n_par <= 0 || n_draft < 0 || !tokens) return -1;
    const int T1 = 1 + n_draft, n = n_par * T1;
    std::vector<int32_t> pos((size_t) n), seq((size_t) n);
    for (int s = 0; s < n_par; ++s)
        for (int j = 0; j < T1; ++j) seq[(size_t) s * T1 + j] = s;
    double acc[4] = {0, 0, 0, 0};
    for (int i = 0; i < n_steps; ++i) {
        for (int s = 0; s < n_par; ++s)
            for (int j = 0; j < T1; ++j) pos[(size_t) s * T1 + j] = pos0 + i + j;
        const int rc = llm_decode(c, n, tokens + (size_t) i * n, pos.data(), seq.data(), nullptr);
        if (rc != 0) return rc;
        for (int k = 0; k < 4; ++k) acc[k] += c->timings[k];
        if (n_draft > 0)
            for (int s = 0; s < n_par; ++s) llm_kv_seq_rm(c, s, pos0 + i + 1, -1);
    }
    for (int k = 0; k < 4; ++k) c->timings[k] = acc[k];
    return 0;
}
extern "C" int llm_n_outputs(const struct llm_context * c) { return c->n_outputs; }
extern "C" float * llm_get_logits(struct llm_context * c) { return c->logits_base; }
// llama_get_logits_ith (include/llama.h; the reference reads through it at llama-box/httpserver.hpp:442 and inside
// common_sampler_sample2 -> set_logits, patches/llama.cpp/sampling.patch:58-81): i >= 0 is a POSITION OF THE BATCH and must be one
// whose logits were requested; i < 0 counts output rows from the end (-1 = the last one).  NULL for anything else.
extern "C" float * llm_get_logits_ith(struct llm_context * c, int i) {
    int row;
    if (i < 0) row = c->n_outputs + i;
    else if ((size_t) i < c->output_ids.size()) row = c->output_ids[(size_t) i];
    else return nullptr;
    if (row < 0 || row >= c->n_outputs) return nullptr;
    return c->logits_base + (size_t) row * c->model->n_vocab_l;
}
// common_sampler_sample2 with the greedy chain llama-box builds for temperature 0 (llama_sampler_init_greedy: the FIRST maximal
// logit wins): the host-side consumer of the logits rows the backend delivers.  -1 if position idx has no logits.
extern "C" int32_t llm_sample_greedy(struct llm_context * c, int idx) {
    const float * lg = llm_get_logits_ith(c, idx);
    if (!lg) return -1;
    const int nv = c->model->n_vocab_l;
    int best = 0;
    for (int t = 1; t < nv; ++t) if (lg[t] > lg[best]) best = t;
    return best;
}
// get_token_probabilities (llama-box/httpserver.hpp:440-467): tokens sorted by logit, soft-max over the whole vocabulary; writes the
// top_n leading (id, p) pairs.  Returns the number written, -1 if position idx has no logits.
extern "C" int llm_token_probabilities(struct llm_context * c, int idx, int top_n, int32_t * ids, float * probs) {
    const float * lg = llm_get_logits_ith(c, idx);
    if (!lg) return -1;
    const int nv = c->model->n_vocab_l;
    std::vector<int32_t> order((size_t) nv);
    for (int t = 0; t < nv; ++t) order[(size_t) t] = t;
    std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return lg[a] > lg[b]; });
    const float max_l = lg[order[0]];
    float cum = 0.0f;
    std::vector<float> p((size_t) nv);
    for (int t = 0; t < nv; ++t) { p[(size_t) t] = expf(lg[order[(size_t) t]] - max_l); cum += p[(size_t) t]; }
    const int n = std::min(top_n, nv);
    for (int t = 0; t < n; ++t) { ids[t] = order[(size_t) t]; probs[t] = p[(size_t) t] / cum; }
    return n;
}
extern "C" struct ggml_cgraph * llm_last_graph(struct llm_context * c) { return c->gf; }
// the K (which = 0) or V (1) cache tensor of layer il: what llama.cpp's state save / slot save reads with ggml_backend_tensor_get
extern "C" struct ggml_tensor * llm_context_cache_tensor(struct llm_context * c, int il, int which) {
    if (il < 0 || il >= (int) c->k_l.size()) return nullptr;
    return which ? c->v_l[(size_t) il] : c->k_l[(size_t) il];
}
extern "C" void llm_last_timings(const struct llm_context * c, double out[4]) {
    for (int k = 0; k < 4; ++k) out[k] = c->timings[k];
}
