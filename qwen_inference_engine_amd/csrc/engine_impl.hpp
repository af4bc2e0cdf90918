// engine_impl.hpp — the engine's and the batch's state, shared by the translation units that
// implement the engine tier: engine.hip (the Qwen decoder: prefill + hipGraph-captured decode)
// and engine_layered.hip (models given as a per-layer program: ragged steps of prompt portions
// and single tokens).  Both kinds of batch use the same slots, block table and page pool.
#pragma once

#include "qie_common.hpp"
#include "../../include/qie/qie_engine.h"
#include "qie_index.hpp"
#include "qie_comm.hpp"

#include <vector>

namespace qie {
struct LayeredModel;   // engine_layered.hip
struct LayeredBatch;
}

// Tensor-parallel shard of one rank (tp = 1: the whole model).  Column-parallel
// QKV (by heads) and gate/up (by I), row-parallel O and down, vocab-parallel lm_head;
// embedding, norms and the residual stream are replicated.
// Heads: n_kv_heads % tp == 0 splits both head kinds evenly; otherwise, when
// tp % n_kv_heads == 0, every kv head is replicated on rep = tp / n_kv_heads ranks and
// the G = n_heads / n_kv_heads q heads of its group are split among those ranks as
// evenly as they go (the first G % rep ranks take one more): Qwen2-7B (28 / 4 heads) at
// TP 8 gives q heads 4,3,4,3,... with one kv head each.  Every q head lives
// on exactly one rank, so the row-parallel O all-reduce still sums each head once.
struct TpShard {
    int tp = 1, rank = 0;
    int nq = 0, nkv = 0, ffn = 0, vocab = 0;   // local counts
    int q0 = 0, kv0 = 0;                        // first global q / kv head of this rank
    int64_t vocab0 = 0;                         // first global vocab row of this rank
};

struct qie_engine {
    qie_model_spec spec{};   // the full model
    TpShard sh;              // this rank's shard
    qie_comm* comm = nullptr;
    qie_engine_opts opts{};
    hipStream_t stream = nullptr;
    void* arena = nullptr;
    size_t arena_bytes = 0;
    qie_index* index = nullptr;
    std::vector<qie_layer_weights> layers;
    qie_model_weights w{};
    bool have_weights = false;
    bool fp8 = false;            // linear weights are e4m3 + row scales (fp8_arena)
    bool fp8_t16 = false;        // ... and the decode projections in the 16-row tiled layout
    bool fp8_t16_head = false;   // ... and the lm_head too
    // fp8 engines: the same (dequantised) layer weights as bf16, in place in the arena —
    // prefill's MFMA GEMMs read these (compute-bound: the LDS-DMA bf16 kernel), decode's
    // bandwidth-bound GEMVs the fp8 codes; both compute the one dequantised model
    std::vector<qie_layer_weights> layers_pf;
    void* fp8_arena = nullptr;
    float* rope_cos = nullptr;
    float* rope_sin = nullptr;
    int rope_rows = 0;
    qie::LayeredModel* lm = nullptr;   // layered engines (engine_layered.hip): architecture + weights
};

struct qie_batch {
    qie_engine* e = nullptr;
    qie::LayeredBatch* lb = nullptr;   // batches of a layered engine: kc is the latent-row pool, vc unused
    int B = 0, max_ctx = 0;
    uint16_t* kc = nullptr;
    uint16_t* vc = nullptr;
    int64_t seq_stride = 0;
    int run_pad = 0;             // contiguous: run = max_ctx + run_pad tokens (dev A/B)
    int32_t* d_pos = nullptr;
    float* d_rope_cur = nullptr;   // [B][rope_cur_stride(hd)]: RoPE row of each slot's current position
    int32_t* d_step = nullptr;
    int32_t* d_hist = nullptr;
    int32_t* d_ids = nullptr;
    unsigned long long* d_keys = nullptr;
    uint16_t* x_res = nullptr;
    uint16_t* qkv = nullptr;
    uint16_t* q = nullptr;
    uint16_t* att = nullptr;
    uint16_t* h = nullptr;
    uint16_t* xn = nullptr;     // [B][H] RMS-normed rows feeding the batched (B >= 2) projections
    uint16_t* logits = nullptr;
    void* attn_ws = nullptr;
    void* dec_ws = nullptr;     // fused decode attention: split partials + zeroed counters
    void* samp_ws = nullptr;
    // tensor parallel: fp32 partials of the row-parallel projections, gathered logits
    float* part = nullptr;            // [B][H]
    uint16_t* logits_full = nullptr;  // [B][V]
    uint16_t* gather_tmp = nullptr;   // [tp][B][V/tp]
    float* pf_part = nullptr;         // [pf_rows][H]
    std::vector<int32_t> h_pos;
    // prefill scratch
    int64_t pf_rows = 0;
    uint16_t *pf_x = nullptr, *pf_hn = nullptr, *pf_qkv = nullptr, *pf_q = nullptr, *pf_att = nullptr,
             *pf_h = nullptr;
    int32_t *pf_pos = nullptr, *pf_ids = nullptr;
    uint8_t *pf_q8 = nullptr, *pf_e8 = nullptr;   // fp8 prefill (opts.prefill_fp8): codes [rows][max K], exps [rows]
    void* pf_attn_ws = nullptr;
    int64_t pf_attn_ws_bytes = 0;   // the split workspace depends on n (short prompts split), not on n <= pf_rows
    // paged KV (qie_batch_create_paged): pool pages of page_tokens tokens, block table
    // [B][max_pages] on device and host, free list, pages held per slot
    int page_tokens = 0, max_pages = 0, n_pages = 0;
    int32_t* d_table = nullptr;
    std::vector<int32_t> h_table, free_pages, held;
    std::vector<char> idle;
    bool table_dirty = false;
    // decode graph
    hipGraphExec_t gexec = nullptr;
    qie_sampling gs{};
    bool graph_ok = false;
    // qie_batch_debug_step: while set, the decode enqueue copies the residual stream after every
    // attention block and every MLP block into dbg_x ([2L + 1][B][H] bf16; slot 0 = the input)
    uint16_t* dbg_x = nullptr;
    // decode structure (qie_batch_set_decode_mode): 0 = five launches per layer, 1 = the whole
    // layer stack as one persistent launch (k_persist.hip).  pk_mem: hand-off granules, then the
    // step epoch and the error word (zeroed once; the finalize kernel advances the epoch)
    int decode_mode = 0;
    void* pk_mem = nullptr;
    qie_layer_weights* d_layers = nullptr;
    void* d_attp = nullptr;      // the attention role's parameters per layer (persist_attn_table)
    unsigned long long* pk_ts = nullptr;   // qie_batch_pk_trace: phase timestamps [cu][layer][slots]
};


namespace qie {
// hipMalloc of at least 16 bytes
int dmalloc(void** p, size_t bytes);
// Page pool of a paged batch (host side, deterministic): take pages so that slot `seq` holds
// positions [0, ntok) (all-or-nothing), return a slot's pages, upload the block table when it
// changed.
int ensure_pages(qie_batch* b, int seq, int64_t ntok);
void drop_pages(qie_batch* b, int seq);
int flush_table(qie_batch* b);
// engine_layered.hip: the parts of the engine tier's shared entry points that differ for a
// layered engine
void layered_engine_destroy(qie_engine* e);
int layered_batch_create(qie_engine* e, int32_t batch, int32_t max_ctx, int32_t page_tokens, int32_t n_pages,
                         qie_batch** out);
void layered_batch_destroy(qie_batch* b);
}  // namespace qie
