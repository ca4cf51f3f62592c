// Paged causal attention for arbitrary head sizes (key size `dim`, value size `vdim`, grouped query heads), bf16 or fp32 cache,
// with the score modifiers of recent decoder designs as PARAMETERS (GeneralAttnParams), each off at its neutral value:
//   * query temperature by position: score *= 1 + coef * ln(floor((p + 1) / every) + 1)          (coef = 0: off)
//   * soft cap:                      score  = cap * tanh(score / cap)                               (cap <= 0: off)
//   * attention sink:                the softmax denominator also holds exp(sink[head]): a learned logit with no key and no value,
//                                    neither scaled nor capped                                      (sink = nullptr: off)
// Scores, soft-max weights and the output accumulation are fp32 whatever the cache holds.
//
// One launch serves every row of a forward, prefill portions and decoded tokens alike: row t belongs to sequence row_seq[t] at
// position row_pos[t] and sees the cache entries 0 .. row_pos[t] of that sequence (its own key was stored before the launch).
//   * row kernel : one wave per (row, query head, key split); lanes own keys for the scores and value channels for the output.
//                  The decode path (few rows, long contexts: split keys + merge kernel) and the fp32 path.
//   * tile kernel: bf16 prefill on the matrix cores -- 64 query rows of one sequence x one query head per workgroup, 64-key cache
//                  blocks through LDS, S = Q K^T and O += P V as v_mfma_f32_16x16x32_bf16, online soft-max in fp32.
#include "tm_kernels.h"

namespace tmk {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ float ga_wave_max(float v)
{
    return group_max<64>(v);
}
__device__ __forceinline__ float ga_wave_sum(float v)
{
    return group_sum<64>(v);
}

__device__ __forceinline__ float ga_query_temp(const GeneralAttnParams& p, int pos)
{
    if (p.qtemp_coef == 0.f) {
        return 1.f;
    }
    const float steps = (float)floor((double)(pos + 1) / (double)p.qtemp_every);
    return 1.f + p.qtemp_coef * logf(steps + 1.f);
}

__device__ __forceinline__ float ga_modify(const GeneralAttnParams& p, float dot, float qscale)
{
    float s = dot * qscale;
    if (p.softcap > 0.f) {
        s = p.softcap * tanhf(s / p.softcap);
    }
    return s;
}

template<class T>
__device__ __forceinline__ float ga_dot(const T* __restrict__ k, const float* __restrict__ q, int D)
{
    float acc = 0.f;
    if constexpr (sizeof(T) == 2) {
        if ((D & 7) == 0) {
            for (int d = 0; d < D; d += 8) {
                const bf16x8 v = *(const bf16x8*)(k + d);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    acc = fmaf((float)v[i], q[d + i], acc);
                }
            }
            return acc;
        }
    }
    else {
        if ((D & 3) == 0) {
            for (int d = 0; d < D; d += 4) {
                const floatx4 v = *(const floatx4*)(k + d);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc = fmaf(v[i], q[d + i], acc);
                }
            }
            return acc;
        }
    }
    for (int d = 0; d < D; ++d) {
        acc = fmaf((float)k[d], q[d], acc);
    }
    return acc;
}

constexpr int kGaMaxDim = 256;  // key / value size limit of the row kernel (q in LDS, four value channels per lane)

// grid (rows, ceil(q_heads / 4), splits), 256 threads: wave w -> head blockIdx.y * 4 + w
template<class T>
__global__ __launch_bounds__(256) void attn_rows_kernel(GeneralAttnParams p)
{
    __shared__ float qs[4][kGaMaxDim];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.x, h = blockIdx.y * 4 + wave, sp = blockIdx.z;
    if (h >= p.q_heads) {
        return;
    }
    const int D = p.dim, V = p.vdim;
    const int s = p.row_seq[t], pos = p.row_pos[t];
    const int g = h / (p.q_heads / p.kv_heads);
    const uint64_t* table = p.block_ptrs + (size_t)(p.seq_slot ? p.seq_slot[s] : s) * p.block_stride;
    const T* q = (const T*)p.q + (size_t)t * p.ldq + (size_t)h * D;
    for (int d = lane; d < D; d += 64) {
        qs[wave][d] = (float)q[d];
    }
    const float qscale = p.scale * ga_query_temp(p, pos);
    const int   nkeys = pos + 1, nblk = (nkeys + p.block_len - 1) / p.block_len;
    const int   per = (nblk + p.splits - 1) / p.splits;
    const int   b0 = sp * per, b1 = min(nblk, b0 + per);
    float m = -1e30f, l = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
    // LDS writes of this wave are read by this wave only: a wave barrier is enough
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int b = b0; b < b1; ++b) {
        const char* base = (const char*)table[b] + p.layer_offset;
        const T*    kb   = (const T*)base + (size_t)g * p.block_len * D;
        const T*    vb   = (const T*)(base + p.v_offset) + (size_t)g * p.block_len * V;
        const int   n    = min(p.block_len, nkeys - b * p.block_len);
        for (int j0 = 0; j0 < n; j0 += 64) {
            const int  j     = j0 + lane;
            const bool valid = j < n;
            float      sc    = -1e30f;
            if (valid) {
                sc = ga_modify(p, ga_dot<T>(kb + (size_t)j * D, qs[wave], D), qscale);
            }
            const float m_new = fmaxf(m, ga_wave_max(sc));
            const float alpha = __expf(m - m_new);
            const float pj    = valid ? __expf(sc - m_new) : 0.f;
            l                 = l * alpha + ga_wave_sum(pj);
            m                 = m_new;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                o[c] *= alpha;
            }
            const int cnt = min(64, n - j0);
            for (int jj = 0; jj < cnt; ++jj) {
                const float w  = __shfl(pj, jj);
                const T*    vr = vb + (size_t)(j0 + jj) * V;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int v = lane + 64 * c;
                    if (v < V) {
                        o[c] = fmaf(w, (float)vr[v], o[c]);
                    }
                }
            }
        }
    }
    if (p.splits == 1) {
        float inv;
        if (p.sink) {
            const float sk = p.sink[h], mf = fmaxf(m, sk), a = __expf(m - mf);
            inv            = a / (l * a + __expf(sk - mf));
        }
        else {
            inv = 1.f / l;
        }
        T* out = (T*)p.out + (size_t)t * p.ldo + (size_t)h * V;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int v = lane + 64 * c;
            if (v < V) {
                out[v] = (T)(o[c] * inv);
            }
        }
        return;
    }
    float* po = p.partial_o + (((size_t)t * p.q_heads + h) * p.splits + sp) * V;
    float* pm = p.partial_ml + (((size_t)t * p.q_heads + h) * p.splits + sp) * 2;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int v = lane + 64 * c;
        if (v < V) {
            po[v] = o[c];
        }
    }
    if (lane == 0) {
        pm[0] = m;
        pm[1] = l;
    }
}

// merge of the key splits (+ the sink): grid (rows, q_heads), 64 threads
template<class T>
__global__ __launch_bounds__(64) void attn_rows_merge_kernel(GeneralAttnParams p)
{
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, V = p.vdim;
    const float* pm = p.partial_ml + ((size_t)t * p.q_heads + h) * p.splits * 2;
    const float* po = p.partial_o + ((size_t)t * p.q_heads + h) * p.splits * V;
    float        mf = p.sink ? p.sink[h] : -1e30f;
    for (int s = 0; s < p.splits; ++s) {
        mf = fmaxf(mf, pm[s * 2]);
    }
    float l = p.sink ? __expf(p.sink[h] - mf) : 0.f;
    float o[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < p.splits; ++s) {
        const float a = __expf(pm[s * 2] - mf);
        l += a * pm[s * 2 + 1];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int v = lane + 64 * c;
            if (v < V) {
                o[c] = fmaf(a, po[(size_t)s * V + v], o[c]);
            }
        }
    }
    T* out = (T*)p.out + (size_t)t * p.ldo + (size_t)h * V;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int v = lane + 64 * c;
        if (v < V) {
            out[v] = (T)(o[c] / l);
        }
    }
}

size_t general_attention_workspace_bytes(int rows, int q_heads, int vdim, int splits)
{
    return (size_t)rows * q_heads * splits * (vdim + 2) * sizeof(float);
}

int launch_general_attention_rows(const GeneralAttnParams& p, hipStream_t st)
{
    TM_REQUIRE(p.rows >= 0 && p.q_heads >= 1 && p.kv_heads >= 1 && p.q_heads % p.kv_heads == 0, "attention: head counts");
    TM_REQUIRE(p.dim >= 1 && p.dim <= kGaMaxDim && p.vdim >= 1 && p.vdim <= kGaMaxDim, "attention: 1 <= dim, vdim <= 256");
    TM_REQUIRE(p.block_len >= 1 && p.splits >= 1 && (p.splits == 1 || (p.partial_o && p.partial_ml)), "attention: splits / workspace");
    TM_REQUIRE(p.elem_bytes == 2 || p.elem_bytes == 4, "attention: bf16 or fp32");
    TM_REQUIRE(p.qtemp_coef == 0.f || p.qtemp_every > 0.f, "attention: query temperature period");
    if (p.rows == 0) {
        return 0;
    }
    const dim3 grid(p.rows, (p.q_heads + 3) / 4, p.splits);
    if (p.elem_bytes == 2) {
        attn_rows_kernel<__bf16><<<grid, 256, 0, st>>>(p);
    }
    else {
        attn_rows_kernel<float><<<grid, 256, 0, st>>>(p);
    }
    TM_HIP_CHECK(hipGetLastError());
    if (p.splits > 1) {
        if (p.elem_bytes == 2) {
            attn_rows_merge_kernel<__bf16><<<dim3(p.rows, p.q_heads), 64, 0, st>>>(p);
        }
        else {
            attn_rows_merge_kernel<float><<<dim3(p.rows, p.q_heads), 64, 0, st>>>(p);
        }
        TM_HIP_CHECK(hipGetLastError());
    }
    return 0;
}

int launch_general_attention(const GeneralAttnParams& p, bool prefill, hipStream_t st)
{
    (void)prefill;
    return launch_general_attention_rows(p, st);
}

}  // namespace tmk
