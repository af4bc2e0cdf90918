// k_layered.hpp — launchers of the layered-model kernels (k_layered.hip).  Host functions take
// a stream, never allocate or synchronise, and return 0 or an error with qie_last_error() text.
#pragma once

#include "qie_common.hpp"

namespace qie {
namespace lay {

// y[m, n] = sum_k A[m, k] W[n, k] (+ batch z: A + z sA, W + z sW, Y + z sY).  A fp32, rounded to
// bf16 on load when round_a; W fp32 or bf16 words; Y fp32.  grp_off (device, batch + 1 entries):
// batch z covers rows [grp_off[z], grp_off[z + 1]) of A and Y (M is then the largest row count a
// group can have).  Three kernels by shape: up to 32 rows a column-per-wave kernel, many rows of a
// bf16 model (mfma) MFMA tiles from memory, else 64 x 64 fp32 tiles through LDS; an element's sum
// never depends on what else the launch holds, only on which of the three ran.
struct LinearP {
    const float* A;
    int64_t lda;
    const void* W;
    int64_t ldw;
    float* Y;
    int64_t ldy;
    int M, N, K, batch;
    int64_t sA, sW, sY;
    int round_a;
    const int32_t* grp_off;
    int mfma;   // bf16 weights, many rows: the direct MFMA kernel may take the product (batched / grouped forms)
};
int linear(const LinearP& p, bool w_f32, hipStream_t st);

// Paged latent cache: page p at pool + p * page_stride elements; inside a page the rows of one
// caching layer start at layer_off and are D = R + rot wide: [c (R) | rotated shared key (rot)].
// Token t of slot s is row t % page_tokens of page table[s * max_pages + t / page_tokens].
struct LatentCache {
    void* pool;
    int64_t page_stride;
    const int32_t* table;
    int page_tokens, max_pages;
};

struct LatentPostP {
    float* proj;          // [T][ld]: q heads, then (own_kv) the compressed row and the shared key part
    int64_t ld;
    const int32_t* row_slot;
    const int32_t* row_pos;
    int heads, dim, rot, rot_dims, R, own_kv;
    const float* norm_w;  // [R]
    float eps;
    const float* rope_cos;   // [positions][rot_dims / 2]
    const float* rope_sin;
    LatentCache cache;
    int64_t layer_off;
    int interleaved;      // bf16 caches: also write the key-interleaved copy of c that follows the rows
};
int latent_post(const LatentPostP& p, bool cache_f32, int T, hipStream_t st);

struct LatentAttnP {
    const float* q_abs;   // [T][heads][R]
    const float* proj;    // rotated query parts are read from the projection rows
    int64_t ld;
    const int32_t* row_slot;
    const int32_t* row_pos;
    int heads, dim, rot, R, window;
    float scale;
    LatentCache cache;
    int64_t layer_off;
    float* out;           // [T][heads][R]
};
int latent_attention(const LatentAttnP& p, bool cache_f32, int T, hipStream_t st);

// The matrix-core form (k_latent_attn.hip; bf16 cache rows followed, per caching layer and page,
// by the key-interleaved copy of c: element ((t % page_tokens) / 4 * R + r) * 4 + t % 4).  A row
// group is up to 16 (token, head) rows of consecutive tokens of one slot: {first packed row,
// tokens, first head, heads per token}.  S splits over the keys; part_o [groups * S][16][R] and
// part_ml [groups * S][16][2] are scratch.
struct LatentAttnMfmaP {
    const float* q_abs;
    const float* proj;
    int64_t ld;
    const int32_t* row_slot;
    const int32_t* row_pos;
    const int4* groups;
    int n_groups, S;
    int heads, dim, rot, R, window;
    float scale;
    LatentCache cache;
    int64_t layer_off;
    float* part_o;
    float* part_ml;
    float* out;           // [T][heads][R]
};
// Row groups a wave takes together: the group list of a step holds, per entry, a multiple of
// kLatentQG groups (padded with empty groups {row, 0, 0, 1}), and consecutive groups of a unit
// belong to one slot.
constexpr int kLatentQG = 1;   // 2 measured slower at kv_rank 256 (one wave per SIMD), and spills at 512
bool latent_attention_mfma_fits(int R, int rot);
int latent_attention_mfma(const LatentAttnMfmaP& p, hipStream_t st);

// The producers below also write the bf16 image of their result when the *_bf pointer is set
// (bf16 engines: the next product reads it; no separate rounding pass).
int embed_rows(const void* E, bool w_f32, const int32_t* tok, float* out, uint16_t* out_bf, int T, int W, int vocab,
               hipStream_t st);
int head_gate(float* v, uint16_t* v_bf, const float* proj, int64_t ld, int g_col, int heads, int vd, int T, hipStream_t st);
// y = (x ? x : 0) + gain * v / sqrt(mean(v^2) + eps), rows of W
int postnorm_add(const float* x, const float* v, float* y, uint16_t* y_bf, int T, int W, float gain, float eps, hipStream_t st);
int final_rows(const float* x, const int32_t* rows, float* out, uint16_t* out_bf, int n, int W, float gain, float eps,
               hipStream_t st);
int depth_mix(const float* stack, int64_t stride, const float* a, int n, float* x, uint16_t* x_bf, int64_t count, hipStream_t st);
int silu_mul(const float* gu, float* a, uint16_t* a_bf, int64_t M, int ff, hipStream_t st);
int route_sigmoid_topk(const float* y, const void* Wr, bool w_f32, int T, int W, int E, int top, int32_t* sel, float* score,
                       hipStream_t st);
int moe_group(const int32_t* sel, int n, int E, int32_t* cnt, int32_t* off, int32_t* slot_of, hipStream_t st);
int moe_gather(const float* y, const float* score, const int32_t* slot_of, int T, int top, int W, float* xg, uint16_t* xg_bf,
               hipStream_t st);
int moe_combine(const float* yd, const int32_t* slot_of, int T, int top, int W, float* f, hipStream_t st);
int argmax_rows(const float* x, int M, int64_t V, int32_t* ids, hipStream_t st);
int rows_to_bf16(const float* x, uint16_t* y, int64_t n, hipStream_t st);
int rows_to_bf16_strided(const float* x, int64_t ldx, uint16_t* y, int64_t ldy, int64_t M, int K, hipStream_t st);
int bf16_to_f32(const uint16_t* x, float* y, int64_t n, hipStream_t st);

}  // namespace lay
}  // namespace qie
