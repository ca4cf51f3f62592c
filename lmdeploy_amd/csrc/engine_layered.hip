// Layer-list model family on the engine: a decoder given as a list of residual blocks (tm_layered_config), each with its mixer, the
// mixer's sizes and constants and its feed-forward.  Everything around the layer loop is the engine's own: block pool and block tables,
// the batch description of forward() (decode / prefill / mixed), the scheduler, sampling, graph capture of the decode step.
//
// Per layer (weights of layer `src`, cache of the layer itself):
//   h1, h2   = norm1(x), norm2(x)                    one launch, one statistic (launch_rmsnorm_f32)
//   [q|k|v]  = h1 . Wqkv^T                           one GEMM over the concatenated projections
//   K, V    -> paged cache; attention -> cat[:, 0 : heads * vdim]
//   cat[:, heads * vdim :] = act(h2 . Wup^T)         activation in the GEMM epilogue
//   x       += residual_mult * (cat . [Wo | Wdown]^T)   ONE GEMM over the concatenated inputs closes the block in its epilogue
// The residual stream x is fp32; h, q, k, v, cat and the cache are bf16 (TM_DTYPE_BF16) or fp32 (TM_DTYPE_F32).
#include "engine_internal.h"

namespace tmk {

__global__ void fill_normal_bf16_kernel(uint16_t* out, size_t n, float mean, float stddev, uint64_t seed)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    uint64_t z = (i + 1) * 0x9E3779B97F4A7C15ull + seed * 0xD1B54A32D192ED03ull;
    z          = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z          = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    const float u1 = ((float)(uint32_t)(z >> 40) + 1.0f) * (1.0f / 16777217.0f);
    const float u2 = (float)(uint32_t)((z >> 8) & 0xffffffu) * (1.0f / 16777216.0f);
    const float v  = mean + stddev * sqrtf(-2.0f * __logf(u1)) * __cosf(6.283185307179586f * u2);
    const __bf16 b = (__bf16)v;
    out[i]         = __builtin_bit_cast(uint16_t, b);
}

// checkpoint bf16 vector -> fp32 (norm weights, sinks)
__global__ void bf16_to_f32_kernel(float* out, const uint16_t* in, size_t n)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        out[i] = __builtin_bit_cast(float, (uint32_t)in[i] << 16);
    }
}

__global__ void iota_kernel(int* out, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        out[i] = i;
    }
}

static std::string lname(int i, const char* t)
{
    return "l" + std::to_string(i) + "." + t;
}

static int to_f32(tm_engine* e, const std::string& name, size_t n, float** out)
{
    Slot& s = e->slots[name];
    TM_REQUIRE(s.filled, "weight not loaded: " + name);
    TM_TRY(dmalloc(out, n));
    bf16_to_f32_kernel<<<(n + 255) / 256, 256, 0, e->stream>>>(*out, (const uint16_t*)s.dev, n);
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

static int place(tm_engine* e, DenseWeight& d, int row0, int col0, const std::string& name, int rows, int cols)
{
    Slot& s = e->slots[name];
    TM_REQUIRE(s.filled, "weight not loaded: " + name);
    return dense_weight_place(d, row0, col0, s.dev, rows, cols, e->stream);
}

int layered_process_weights(tm_engine* e)
{
    LayeredModel&            lm = *e->lm;
    const tm_layered_config& c  = lm.cfg;
    const int                dt = c.dtype == TM_DTYPE_F32 ? kDenseF32 : kDenseBf16;
    const int                W  = c.width;
    for (int i = 0; i < c.n_layers; ++i) {
        LmLayer& L = lm.layers[i];
        if (L.src != i) {
            continue;
        }
        const tm_layer_spec& s = L.spec;
        TM_TRY(dense_weight_alloc(L.qkv, W, L.n_q + L.n_k + L.n_v, dt, e->stream));
        TM_TRY(place(e, L.qkv, 0, 0, lname(i, "mix.q"), L.n_q, W));
        TM_TRY(place(e, L.qkv, L.n_q, 0, lname(i, "mix.k"), L.n_k, W));
        TM_TRY(place(e, L.qkv, L.n_q + L.n_k, 0, lname(i, "mix.v"), L.n_v, W));
        TM_TRY(dense_weight_alloc(L.out, L.n_att + (s.mlp ? s.ff : 0), W, dt, e->stream));
        // [o | down] along K: the checkpoint rows have their own lengths, each part is placed at its column offset
        TM_TRY(place(e, L.out, 0, 0, lname(i, "mix.o"), W, L.n_att));
        TM_TRY(to_f32(e, lname(i, "norm1"), W, &L.norm1));
        if (s.sink) {
            TM_TRY(to_f32(e, lname(i, "mix.sink"), s.heads, &L.sink));
        }
        if (s.mlp) {
            TM_TRY(dense_weight_alloc(L.up, W, s.ff, dt, e->stream));
            TM_TRY(place(e, L.up, 0, 0, lname(i, "mlp.up"), s.ff, W));
            TM_TRY(place(e, L.out, 0, L.n_att, lname(i, "mlp.down"), W, s.ff));
            TM_TRY(to_f32(e, lname(i, "norm2"), W, &L.norm2));
        }
    }
    for (int i = 0; i < c.n_layers; ++i) {  // borrowed weights
        LmLayer& L = lm.layers[i];
        if (L.src != i) {
            const LmLayer& S = lm.layers[L.src];
            L.qkv = S.qkv, L.up = S.up, L.out = S.out, L.norm1 = S.norm1, L.norm2 = S.norm2, L.sink = S.sink;
        }
    }
    TM_TRY(dense_weight_alloc(lm.head, W, c.vocab, dt, e->stream));
    TM_TRY(place(e, lm.head, 0, 0, "head", c.vocab, W));
    TM_TRY(to_f32(e, "final.norm", W, &lm.final_norm));
    {
        Slot& s = e->slots["embed"];
        TM_REQUIRE(s.filled, "weight not loaded: embed");
        if (c.dtype == TM_DTYPE_F32) {
            float* f = nullptr;
            TM_TRY(dmalloc(&f, (size_t)c.vocab * W));
            bf16_to_f32_kernel<<<((size_t)c.vocab * W + 255) / 256, 256, 0, e->stream>>>(f, (const uint16_t*)s.dev, (size_t)c.vocab * W);
            TM_HIP_CHECK(hipGetLastError());
            lm.embed = f;
        }
        else {
            lm.embed = s.dev;  // used in place
            s.dev    = nullptr;
        }
    }
    TM_HIP_CHECK(hipStreamSynchronize(e->stream));
    for (auto& kv : e->slots) {  // staging is no longer needed
        if (kv.second.dev) {
            (void)hipFree(kv.second.dev);
            kv.second.dev = nullptr;
        }
    }
    e->weights_ready = true;
    return 0;
}

int layered_init_synthetic(tm_engine* e, uint64_t seed)
{
    uint64_t sd = seed * 1000003ull + 29;
    for (auto& kv : e->slots) {
        Slot&             s = kv.second;
        const std::string& n = kv.first;
        if (!s.dev) {
            TM_HIP_CHECK(hipMalloc(&s.dev, s.bytes));
        }
        const size_t cnt  = (size_t)s.bytes / 2;
        const bool   vec  = n.find("norm") != std::string::npos || n.find("sink") != std::string::npos;
        // matrices: N(0, 1 / in_features) keeps every projection's output at the scale of its input; vectors: small, around zero
        float        stdv = 0.02f;
        if (!vec && n != "embed") {
            const LayeredModel& lm = *e->lm;
            int                 K  = lm.cfg.width;
            const size_t        dot = n.rfind('.');
            const std::string   leaf = dot == std::string::npos ? n : n.substr(dot + 1);
            if (leaf == "o" || leaf == "down") {
                K = (int)(cnt / lm.cfg.width);
            }
            stdv = 1.0f / std::sqrt((float)K);
        }
        else if (n == "embed") {
            stdv = 1.0f;
        }
        fill_normal_bf16_kernel<<<(cnt + 255) / 256, 256, 0, e->stream>>>((uint16_t*)s.dev, cnt, 0.f, stdv, ++sd);
        TM_HIP_CHECK(hipGetLastError());
        s.filled = true;
    }
    TM_HIP_CHECK(hipStreamSynchronize(e->stream));
    return 0;
}

template<class T>
static int lm_alloc(T** p, size_t n, hipStream_t st)
{
    TM_HIP_CHECK(hipMalloc((void**)p, n * sizeof(T)));
    TM_HIP_CHECK(hipMemsetAsync(*p, 0, n * sizeof(T), st));
    return 0;
}

// start-up allocation of a layer-list engine: activation buffers, batch state, block pool (the engine's own fields, so that the
// static batch, continuous batching and the sampler run unchanged)
int layered_start(tm_engine* e)
{
    LayeredModel&            lm = *e->lm;
    const tm_layered_config& m  = lm.cfg;
    const tm_engine_config&  c  = e->cfg;
    hipStream_t              st = e->stream;
    const int                B  = c.max_batch_size;
    e->max_blocks_per_seq = (c.session_len + c.cache_block_seq_len - 1) / c.cache_block_seq_len;
    e->max_tokens         = std::max(B, std::max(64, c.max_prefill_token_num));
    const size_t T        = e->max_tokens;
    // cache block: every layer run has its keys [kv_heads][block_len][dim] and, behind them, its values transposed [kv_heads][vdim][block_len]
    int64_t off = 0;
    int     max_qkv = 0, max_cat = 0, max_vdim = 0, max_heads = 0;
    for (LmLayer& L : lm.layers) {
        L.kv_offset = off;
        L.v_offset  = (int64_t)L.n_k * c.cache_block_seq_len * lm.elem;
        off += (int64_t)(L.n_k + L.n_v) * c.cache_block_seq_len * lm.elem;
        off         = (off + 15) / 16 * 16;
        max_qkv     = std::max(max_qkv, L.qkv.N);
        max_cat     = std::max(max_cat, L.out.Kp);
        max_vdim    = std::max(max_vdim, L.spec.vdim);
        max_heads   = std::max(max_heads, L.spec.heads);
    }
    e->block_bytes = off;
    lm.ldw   = (m.width + 31) / 32 * 32;
    lm.ldqkv = (max_qkv + 31) / 32 * 32;
    lm.ldcat = max_cat;
    lm.ldv16 = e->vocab_local;
    lm.max_logit_rows = (int)std::max<size_t>(B, std::min<size_t>(T, 1024));
    TM_TRY(lm_alloc(&lm.d_res, T * m.width, st));
    TM_TRY(lm_alloc((char**)&lm.d_h1, T * lm.ldw * lm.elem, st));
    TM_TRY(lm_alloc((char**)&lm.d_h2, T * lm.ldw * lm.elem, st));
    TM_TRY(lm_alloc((char**)&lm.d_qkv, T * lm.ldqkv * lm.elem, st));
    TM_TRY(lm_alloc((char**)&lm.d_cat, T * lm.ldcat * lm.elem, st));
    TM_TRY(lm_alloc((char**)&lm.d_hn, (size_t)lm.max_logit_rows * lm.ldw * lm.elem, st));
    TM_TRY(lm_alloc(&lm.d_logits_f32, (size_t)lm.max_logit_rows * m.vocab, st));
    TM_TRY(lm_alloc(&lm.d_row_seq, T, st));
    TM_TRY(lm_alloc(&lm.d_row_pos, T, st));
    TM_TRY(lm_alloc(&lm.d_want, T, st));
    TM_TRY(lm_alloc(&lm.d_iota, T, st));
    TM_TRY(lm_alloc(&lm.d_seq_slot, (size_t)B, st));
    TM_TRY(lm_alloc(&lm.d_step_ids, T, st));
    TM_TRY(lm_alloc(&lm.d_step_cu_q, (size_t)B + 1, st));
    TM_TRY(lm_alloc(&lm.d_step_k_len, (size_t)B, st));
    iota_kernel<<<(T + 255) / 256, 256, 0, st>>>(lm.d_iota, (int)T);
    TM_HIP_CHECK(hipGetLastError());
    // decode rows split their keys so that a few long sequences still fill the device: >= 4 cache blocks per split at full length
    lm.decode_splits = std::min(8, std::max(1, e->max_blocks_per_seq / 4));
    lm.attn_ws_bytes = general_attention_workspace_bytes(B, max_heads, max_vdim, lm.decode_splits);
    TM_HIP_CHECK(hipMalloc((void**)&lm.d_attn_ws, lm.attn_ws_bytes));

    // the engine's batch state (same fields as every other model family)
    TM_TRY(lm_alloc(&e->d_logits, (size_t)B * e->vocab_local, st));
    TM_TRY(lm_alloc(&e->d_ids, (size_t)B, st));
    TM_TRY(lm_alloc(&e->d_next_ids, (size_t)B, st));
    TM_TRY(lm_alloc(&e->d_k_len, (size_t)B, st));
    TM_TRY(lm_alloc(&e->d_cu_q, (size_t)B + 1, st));
    TM_TRY(lm_alloc(&e->d_cu_q_b, (size_t)B + 1, st));
    TM_TRY(lm_alloc(&e->d_cu_koff, (size_t)B + 1, st));
    TM_TRY(lm_alloc(&e->d_rows, (size_t)B, st));
    TM_TRY(lm_alloc(&e->d_generated, (size_t)B * c.session_len, st));
    TM_TRY(lm_alloc(&e->d_step, (size_t)1, st));
    TM_TRY(lm_alloc(&e->d_prefill_ids, T, st));
    TM_TRY(lm_alloc(&e->d_argmax_val, (size_t)B, st));
    TM_TRY(lm_alloc(&e->d_cand, (size_t)B * 2, st));
    TM_TRY(lm_alloc(&e->d_cand_all, (size_t)B * 2, st));
    TM_TRY(lm_alloc(&e->d_block_ptrs, (size_t)B * e->max_blocks_per_seq, st));
    TM_TRY(lm_alloc(&e->d_cu_block_nums, (size_t)B + 1, st));
    e->kflat_stride = 1 << 30;  // no flatten scratch in this family: the attention kernels read the paged cache

    int64_t blocks = c.cache_blocks;
    if (blocks <= 0) {
        size_t free_b = 0, total_b = 0;
        TM_HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
        const float frac = c.cache_max_entry_count > 0.f ? c.cache_max_entry_count : 0.8f;
        blocks           = (int64_t)((double)free_b * frac / (double)e->block_bytes);
        blocks           = std::min(blocks, (int64_t)B * e->max_blocks_per_seq + 1);
    }
    TM_REQUIRE(blocks >= 1, "no memory for KV blocks");
    if (hipMalloc((void**)&e->pool, (size_t)blocks * e->block_bytes) != hipSuccess) {
        (void)hipGetLastError();
        set_last_error("KV pool allocation failed");
        return TM_OOM;
    }
    TM_HIP_CHECK(hipMemsetAsync(e->pool, 0, (size_t)blocks * e->block_bytes, st));
    e->num_blocks = blocks;
    e->free_blocks.resize(blocks);
    for (int64_t i = 0; i < blocks; ++i) {
        e->free_blocks[i] = (int)(blocks - 1 - i);
    }
    TM_HIP_CHECK(hipStreamSynchronize(st));
    e->started = true;
    return 0;
}

void layered_free(tm_engine* e)
{
    if (!e->lm) {
        return;
    }
    LayeredModel& lm = *e->lm;
    for (size_t i = 0; i < lm.layers.size(); ++i) {
        LmLayer& L = lm.layers[i];
        if (L.src == (int)i) {
            dense_weight_free(L.qkv), dense_weight_free(L.up), dense_weight_free(L.out);
            for (float* p : {L.norm1, L.norm2, L.sink}) {
                if (p) {
                    (void)hipFree(p);
                }
            }
        }
    }
    dense_weight_free(lm.head);
    for (void* p : {(void*)lm.embed, (void*)lm.final_norm, (void*)lm.d_res, lm.d_h1, lm.d_h2, lm.d_qkv, lm.d_cat, lm.d_hn, (void*)lm.d_logits_f32,
                    (void*)lm.d_row_seq, (void*)lm.d_row_pos, (void*)lm.d_iota, (void*)lm.d_want, (void*)lm.d_seq_slot, (void*)lm.d_step_ids,
                    (void*)lm.d_step_cu_q, (void*)lm.d_step_k_len, (void*)lm.d_attn_ws}) {
        if (p) {
            (void)hipFree(p);
        }
    }
}

// ---- forward ------------------------------------------------------------------------------------------------------------------------
static GeneralAttnParams attn_params(tm_engine* e, const LmLayer& L, const LmPart& P)
{
    LayeredModel&     lm = *e->lm;
    GeneralAttnParams p{};
    p.q            = (const char*)lm.d_qkv + (size_t)P.row0 * lm.ldqkv * lm.elem;
    p.out          = (char*)lm.d_cat + (size_t)P.row0 * lm.ldcat * lm.elem;
    p.ldq          = lm.ldqkv;
    p.ldo          = lm.ldcat;
    p.rows         = P.rows;
    p.row_seq      = lm.d_row_seq + P.row0;
    p.row_pos      = lm.d_row_pos + P.row0;
    p.seq_slot     = P.seq_slot;
    p.block_ptrs   = P.block_ptrs;
    p.block_stride = e->max_blocks_per_seq;
    p.layer_offset = L.kv_offset;
    p.v_offset     = L.v_offset;
    p.block_len    = e->cfg.cache_block_seq_len;
    p.elem_bytes   = lm.elem;
    p.q_heads      = L.spec.heads;
    p.kv_heads     = L.spec.kv_heads;
    p.dim          = L.spec.dim;
    p.vdim         = L.spec.vdim;
    p.scale        = L.spec.scale;
    p.softcap      = L.spec.softcap;
    p.qtemp_coef   = L.spec.qtemp_coef;
    p.qtemp_every  = L.spec.qtemp_every;
    p.sink         = L.sink;
    p.nseq         = P.nseq;
    p.max_q_len    = P.max_q_len;
    p.cu_q         = P.cu_q;
    p.k_len        = P.k_len;
    return p;
}

// the layer loop over M rows described by `parts`; leaves the residual stream in lm.d_res
static int layered_layers(tm_engine* e, const int* d_ids, int M, const LmPart* parts, int nparts)
{
    LayeredModel&            lm = *e->lm;
    const tm_layered_config& m  = lm.cfg;
    hipStream_t              st = e->stream;
    TM_REQUIRE(M >= 1 && M <= e->max_tokens, "forward: more rows than max_prefill_token_num");
    for (int i = 0; i < nparts; ++i) {
        const LmPart& P = parts[i];
        TM_TRY(launch_rows_prepare(lm.d_row_seq + P.row0, lm.d_row_pos + P.row0, P.cu_q, P.k_len, P.nseq, P.rows, st));
    }
    TM_PROF(P_EMBED, TM_TRY(launch_embedding_f32(lm.d_res, lm.embed, lm.elem, d_ids, M, m.width, m.vocab, st)));
    const int n_run = lm.debug_layers >= 0 ? std::min(lm.debug_layers, m.n_layers) : m.n_layers;
    for (int li = 0; li < n_run; ++li) {
        const LmLayer&       L = lm.layers[li];
        const tm_layer_spec& s = L.spec;
        TM_PROF(P_RES_NORM, TM_TRY(launch_rmsnorm_f32(lm.d_h1, s.mlp ? lm.d_h2 : nullptr, lm.ldw, lm.elem, lm.d_res, nullptr, L.norm1, L.norm2,
                                                      m.norm_offset, m.norm_eps, M, m.width, st)));
        TM_PROF(P_GEMM_QKV, TM_TRY(launch_dense_linear(L.qkv, lm.d_h1, lm.ldw, lm.d_qkv, lm.ldqkv, M, kDenseStore, 1.f, st)));
        for (int i = 0; i < nparts; ++i) {
            const LmPart&     P = parts[i];
            GeneralAttnParams p = attn_params(e, L, P);
            TM_PROF(P_KV_STORE, TM_TRY(launch_kv_store_general(p.q, lm.ldqkv, L.n_q, L.n_q + L.n_k, p, st)));
            if (P.decode && lm.decode_splits > 1
                && general_attention_workspace_bytes(P.rows, s.heads, s.vdim, lm.decode_splits) <= lm.attn_ws_bytes) {
                p.splits     = lm.decode_splits;
                p.partial_o  = lm.d_attn_ws;
                p.partial_ml = lm.d_attn_ws + (size_t)P.rows * s.heads * p.splits * s.vdim;
            }
            TM_PROF(P_ATTN, TM_TRY(launch_general_attention(p, !P.decode, st)));
        }
        if (s.mlp) {
            TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_dense_linear(L.up, lm.d_h2, lm.ldw, (char*)lm.d_cat + (size_t)L.n_att * lm.elem, lm.ldcat, M,
                                                               kDenseRelu2, 1.f, st)));
        }
        TM_PROF(P_GEMM_O, TM_TRY(launch_dense_linear(L.out, lm.d_cat, lm.ldcat, lm.d_res, m.width, M, kDenseResidAdd, m.residual_mult, st)));
    }
    return 0;
}

// fp32 logits of `n` rows of the residual stream (rows == nullptr: rows 0 .. n-1) -> lm.d_logits_f32 [n][vocab]
static int layered_logits(tm_engine* e, const int* rows, int n)
{
    LayeredModel&            lm = *e->lm;
    const tm_layered_config& m  = lm.cfg;
    TM_REQUIRE(n <= lm.max_logit_rows, "internal: too many logits rows");
    TM_PROF(P_RES_NORM, TM_TRY(launch_rmsnorm_f32(lm.d_hn, nullptr, lm.ldw, lm.elem, lm.d_res, rows, lm.final_norm, nullptr, m.norm_offset,
                                                  m.norm_eps, n, m.width, e->stream)));
    TM_PROF(P_LM_HEAD, TM_TRY(launch_dense_linear(lm.head, lm.d_hn, lm.ldw, lm.d_logits_f32, m.vocab, n, kDenseScaleF32, m.logit_scale, e->stream)));
    return 0;
}

// logits of `n` sequences -> the engine's fp16 logits rows at the batch slots [slot, slot + n) -> logits processors + sampling
static int layered_head(tm_engine* e, const int* rows, int n, int slot, const int* ids_in, const int* cu_q, int ntok, const int* k_len,
                        const int* active)
{
    LayeredModel& lm = *e->lm;
    for (int r0 = 0; r0 < n; r0 += lm.max_logit_rows) {
        const int cnt = std::min(lm.max_logit_rows, n - r0);
        TM_TRY(layered_logits(e, rows + r0, cnt));
        TM_TRY(launch_f32_to_f16_rows(e->d_logits + (size_t)(slot + r0) * e->vocab_local, e->vocab_local, lm.d_logits_f32, cnt, lm.cfg.vocab,
                                      e->stream));
    }
    return sample_rows(e, n, slot, ids_in, cu_q, ntok, k_len, active);
}

// forward() of the engine for this family: the same batch description as every other model (engine_forward.hip)
int layered_forward(tm_engine* e, const int* d_ids, int M, int nseq, bool decode, int max_q_len, int max_k_len, int slot0, const MixedDecode* md)
{
    LayeredModel& lm = *e->lm;
    const int     nd = md ? md->rows : 0;
    TM_REQUIRE(!md || (!decode && nd > 0 && nd < M), "internal: mixed forward");
    LmPart parts[2];
    int    np = 0;
    if (md) {  // the decode rows of every batch slot first, on the decode state's own table
        parts[np++] = LmPart{0, nd, nd, md->cu_q, md->k_len, nullptr, md->block_ptrs, true, 1};
    }
    parts[np++] = LmPart{nd, M - nd, nseq, e->d_cu_q, e->d_k_len, nullptr, e->d_block_ptrs, decode, decode ? 1 : max_q_len};
    TM_TRY(layered_layers(e, d_ids, M, parts, np));
    if (decode) {
        return layered_head(e, lm.d_iota, nseq, slot0, d_ids, nullptr, M, e->d_k_len, nullptr);
    }
    if (md) {
        TM_TRY(layered_head(e, lm.d_iota, nd, 0, d_ids, nullptr, nd, md->k_len, md->active));
    }
    return layered_head(e, e->d_rows, nseq, slot0, d_ids + nd, e->d_cu_q, M - nd, e->d_k_len, nullptr);  // d_rows: last row of every sequence
}

}  // namespace tmk

extern "C" {

int tm_engine_create_layered(tm_engine** out, const tm_engine_config* c, const tm_layered_config* m)
{
    TM_REQUIRE(out && c && m && m->layers, "null pointer");
    TM_REQUIRE(c->tp == 1 && c->rank == 0, "layer-list models run on one GPU (tp = 1)");
    TM_REQUIRE(c->quant_policy == 0, "layer-list models keep the cache in the activation type (quant_policy 0)");
    TM_REQUIRE(c->cache_block_seq_len == 64, "cache_block_seq_len must be 64");
    TM_REQUIRE(c->max_batch_size >= 1 && c->max_batch_size <= 1024 && c->session_len >= 1, "1 <= max_batch_size <= 1024, session_len >= 1");
    TM_REQUIRE(m->width >= 1 && m->vocab >= 1 && m->n_layers >= 1, "width, vocab, layers >= 1");
    TM_REQUIRE(m->dtype == TM_DTYPE_BF16 || m->dtype == TM_DTYPE_F32, "dtype: bf16 | f32");
    TM_REQUIRE(m->norm_eps > 0.f, "norm_eps > 0");
    for (int i = 0; i < m->n_layers; ++i) {
        const tm_layer_spec& s = m->layers[i];
        TM_REQUIRE(s.mixer == TM_MIXER_ATTENTION, "layer " + std::to_string(i) + ": unknown mixer");
        TM_REQUIRE(s.heads >= 1 && s.kv_heads >= 1 && s.heads % s.kv_heads == 0, "layer " + std::to_string(i) + ": heads % kv_heads");
        TM_REQUIRE(s.dim >= 1 && s.dim <= 256 && s.vdim >= 1 && s.vdim <= 256, "layer " + std::to_string(i) + ": 1 <= dim, vdim <= 256");
        TM_REQUIRE(s.mlp == TM_MLP_NONE || (s.mlp == TM_MLP_DENSE && s.ff >= 1 && s.act == TM_ACT_RELU2), "layer " + std::to_string(i) + ": feed-forward");
        TM_REQUIRE(s.qtemp_coef == 0.f || s.qtemp_every > 0.f, "layer " + std::to_string(i) + ": query temperature period");
        TM_REQUIRE(s.weights_of < 0 || (s.weights_of < m->n_layers && s.weights_of != i && m->layers[s.weights_of].weights_of < 0),
                   "layer " + std::to_string(i) + ": weights_of must name a layer with tensors of its own");
        if (s.weights_of >= 0) {
            const tm_layer_spec& o = m->layers[s.weights_of];
            TM_REQUIRE(o.heads == s.heads && o.kv_heads == s.kv_heads && o.dim == s.dim && o.vdim == s.vdim && o.mlp == s.mlp && o.ff == s.ff
                           && o.sink == s.sink,
                       "layer " + std::to_string(i) + ": sizes differ from the layer whose weights it uses");
        }
    }
    TM_HIP_CHECK(hipSetDevice(c->device));
    auto* e = new tm_engine();
    e->cfg  = *c;
    memset(&e->cfg.model, 0, sizeof(e->cfg.model));
    e->cfg.model.hidden = m->width;
    e->cfg.model.layers = m->n_layers;
    e->cfg.model.vocab  = m->vocab;
    e->hidden           = m->width;
    e->vocab_local      = (m->vocab + 7) / 8 * 8;  // fp16 logits rows of the sampler: 16-byte aligned, pad columns never win
    e->q_heads = e->kv_heads = 1;                  // (the decode-split heuristic of the fixed-head-size kernels reads them; unused here)
    e->mixed_steps_on   = !(getenv("TM_MIXED_STEP") && !atoi(getenv("TM_MIXED_STEP")));
    TM_HIP_CHECK(hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking));
    e->lm.reset(new LayeredModel());
    LayeredModel& lm = *e->lm;
    lm.cfg           = *m;
    lm.cfg.layers    = nullptr;
    lm.elem          = m->dtype == TM_DTYPE_F32 ? 4 : 2;
    lm.layers.resize(m->n_layers);
    const int64_t W = m->width;
    for (int i = 0; i < m->n_layers; ++i) {
        LmLayer& L = lm.layers[i];
        L.spec     = m->layers[i];
        L.src      = L.spec.weights_of >= 0 ? L.spec.weights_of : i;
        L.n_q      = L.spec.heads * L.spec.dim;
        L.n_k      = L.spec.kv_heads * L.spec.dim;
        L.n_v      = L.spec.kv_heads * L.spec.vdim;
        L.n_att    = L.spec.heads * L.spec.vdim;
        if (L.src != i) {
            continue;
        }
        e->slots[lname(i, "norm1")].bytes = W * 2;
        e->slots[lname(i, "mix.q")].bytes = W * L.n_q * 2;
        e->slots[lname(i, "mix.k")].bytes = W * L.n_k * 2;
        e->slots[lname(i, "mix.v")].bytes = W * L.n_v * 2;
        e->slots[lname(i, "mix.o")].bytes = W * L.n_att * 2;
        if (L.spec.sink) {
            e->slots[lname(i, "mix.sink")].bytes = (int64_t)L.spec.heads * 2;
        }
        if (L.spec.mlp) {
            e->slots[lname(i, "norm2")].bytes    = W * 2;
            e->slots[lname(i, "mlp.up")].bytes   = W * L.spec.ff * 2;
            e->slots[lname(i, "mlp.down")].bytes = W * L.spec.ff * 2;
        }
    }
    e->slots["embed"].bytes      = W * m->vocab * 2;
    e->slots["final.norm"].bytes = W * 2;
    e->slots["head"].bytes       = W * m->vocab * 2;
    *out = e;
    return 0;
}

int tm_engine_debug_stop_after(tm_engine* e, int layers)
{
    TM_REQUIRE(e && e->lm, "layer-list engine");
    e->lm->debug_layers = layers;
    return 0;
}

int tm_engine_session_open(tm_engine* e, int64_t* session)
{
    TM_REQUIRE(e && session, "null pointer");
    TM_REQUIRE(e->lm, "sessions need a layer-list model");
    if (e->loop_on.load()) {
        set_last_error("the engine thread is running (tm_engine_serve_stop first)");
        return TM_CONFLICT;
    }
    ApiLock lk(e);
    TM_TRY(cb_enter(e));
    if (e->sched->n_active() > e->sched->n_sessions() || e->sched->n_waiting() > 0) {
        set_last_error("queued / running requests exist: sessions and tm_engine_submit do not share a scheduler session");
        return TM_CONFLICT;
    }
    if (e->sched->open_session(session)) {
        set_last_error("no free batch slot");
        return TM_CONFLICT;
    }
    e->lm->sess_len[*session] = 0;
    return 0;
}

int tm_engine_session_close(tm_engine* e, int64_t session)
{
    TM_REQUIRE(e && e->lm && e->sched, "no open session");
    ApiLock lk(e);
    TM_HIP_CHECK(hipStreamSynchronize(e->stream));
    TM_REQUIRE(e->sched->close_session(session) == 0, "unknown session");
    e->lm->sess_len.erase(session);
    return 0;
}

int tm_engine_step_tokens(tm_engine* e, const tm_step_entry* entries, int n_entries, float* host_logits)
{
    TM_REQUIRE(e && entries && n_entries >= 1, "null pointer / no entries");
    TM_REQUIRE(e->lm && e->sched, "no open session");
    ApiLock       lk(e);
    LayeredModel& lm = *e->lm;
    TM_HIP_CHECK(hipSetDevice(e->cfg.device));
    TM_REQUIRE(n_entries <= e->cfg.max_batch_size, "more entries than batch slots");
    // decoded tokens (one row) first, portions after them: two parts of one forward, each on its kind of attention kernel
    std::vector<int> order;
    for (int pass = 0; pass < 2; ++pass) {
        for (int i = 0; i < n_entries; ++i) {
            TM_REQUIRE(entries[i].n_tokens >= 1 && entries[i].tokens, "entry without tokens");
            if ((entries[i].n_tokens == 1) == (pass == 0)) {
                order.push_back(i);
            }
        }
    }
    int need = 0, total = 0, n_dec = 0;
    for (int i = 0; i < n_entries; ++i) {
        const tm_step_entry& en = entries[i];
        auto                 it = lm.sess_len.find(en.session);
        TM_REQUIRE(it != lm.sess_len.end(), "unknown session");
        for (int j = 0; j < i; ++j) {
            TM_REQUIRE(entries[j].session != en.session, "a session appears twice in one step");
        }
        const int nb = e->sched->grow_need(en.session, it->second + en.n_tokens);
        if (nb < 0) {
            set_last_error("session exceeds session_len");
            return TM_TOO_LONG;
        }
        need += nb;
        total += en.n_tokens;
        n_dec += en.n_tokens == 1;
        for (int w = 0; w < en.n_want; ++w) {
            TM_REQUIRE(en.want && en.want[w] >= 0 && en.want[w] < en.n_tokens, "want: index outside the entry's tokens");
        }
    }
    TM_REQUIRE(total <= e->max_tokens, "step brings more tokens than max_prefill_token_num");
    if (need > e->sched->n_free_blocks()) {
        set_last_error("out of KV cache blocks");
        return TM_OOM;
    }
    std::vector<int> ids, cu_q{0}, k_len, slots, want;
    std::vector<int> want_of(n_entries + 1, 0);  // logits rows are returned in ENTRY order: remember where each entry's rows start
    int              max_q = 1;
    std::vector<std::vector<int>> want_rows(n_entries);
    for (int oi : order) {
        const tm_step_entry& en  = entries[oi];
        int&                 len = lm.sess_len[en.session];
        const SchedRequest*  r   = e->sched->find(en.session);
        const size_t         had = r->blocks.size();
        TM_REQUIRE(e->sched->grow(en.session, len + en.n_tokens), "internal: block accounting");
        if (r->blocks.size() > had) {  // new blocks join the session's row of the block table
            std::vector<uint64_t> ptrs;
            for (size_t q = had; q < r->blocks.size(); ++q) {
                ptrs.push_back((uint64_t)(e->pool + (int64_t)r->blocks[q] * e->block_bytes));
            }
            TM_HIP_CHECK(hipMemcpyAsync(e->d_block_ptrs + (size_t)r->slot * e->max_blocks_per_seq + had, ptrs.data(), ptrs.size() * 8,
                                        hipMemcpyHostToDevice, e->stream));
            TM_HIP_CHECK(hipStreamSynchronize(e->stream));
        }
        for (int w = 0; w < en.n_want; ++w) {
            want_rows[oi].push_back((int)ids.size() + en.want[w]);
        }
        ids.insert(ids.end(), en.tokens, en.tokens + en.n_tokens);
        cu_q.push_back((int)ids.size());
        len += en.n_tokens;
        k_len.push_back(len);
        slots.push_back(r->slot);
        max_q = std::max(max_q, en.n_tokens);
    }
    for (int i = 0; i < n_entries; ++i) {
        want.insert(want.end(), want_rows[i].begin(), want_rows[i].end());
    }
    hipStream_t st = e->stream;
    TM_HIP_CHECK(hipMemcpyAsync(lm.d_step_ids, ids.data(), ids.size() * 4, hipMemcpyHostToDevice, st));
    TM_HIP_CHECK(hipMemcpyAsync(lm.d_step_cu_q, cu_q.data(), cu_q.size() * 4, hipMemcpyHostToDevice, st));
    TM_HIP_CHECK(hipMemcpyAsync(lm.d_step_k_len, k_len.data(), k_len.size() * 4, hipMemcpyHostToDevice, st));
    TM_HIP_CHECK(hipMemcpyAsync(lm.d_seq_slot, slots.data(), slots.size() * 4, hipMemcpyHostToDevice, st));
    if (!want.empty()) {
        TM_HIP_CHECK(hipMemcpyAsync(lm.d_want, want.data(), want.size() * 4, hipMemcpyHostToDevice, st));
    }
    LmPart parts[2];
    int    np = 0;
    if (n_dec > 0) {
        parts[np++] = LmPart{0, n_dec, n_dec, lm.d_step_cu_q, lm.d_step_k_len, lm.d_seq_slot, e->d_block_ptrs, true, 1};
    }
    if (n_dec < n_entries) {
        // the portions' description starts at entry n_dec: cu_q values count from row 0 of the forward, the part's rows from n_dec
        parts[np++] = LmPart{n_dec, total - n_dec, n_entries - n_dec, lm.d_step_cu_q + n_dec, lm.d_step_k_len + n_dec, lm.d_seq_slot + n_dec,
                             e->d_block_ptrs, false, max_q};
    }
    int rc = layered_layers(e, lm.d_step_ids, total, parts, np);
    const int V = lm.cfg.vocab;
    for (size_t r0 = 0; rc == 0 && r0 < want.size(); r0 += lm.max_logit_rows) {
        const int cnt = (int)std::min<size_t>(lm.max_logit_rows, want.size() - r0);
        rc            = layered_logits(e, lm.d_want + r0, cnt);
        if (rc == 0) {
            TM_REQUIRE(host_logits, "host_logits is null but logits are wanted");
            TM_HIP_CHECK(hipMemcpyAsync(host_logits + r0 * V, lm.d_logits_f32, (size_t)cnt * V * 4, hipMemcpyDeviceToHost, st));
            TM_HIP_CHECK(hipStreamSynchronize(st));
        }
    }
    TM_HIP_CHECK(hipStreamSynchronize(st));  // the host vectors above are pageable
    return rc;
}

}  // extern "C"
