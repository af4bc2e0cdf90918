// k_latent_attn.hip — sliding-window latent attention on the matrix cores (bf16 cache rows).
//
// Absorbed form: every head of a token scores the SAME cached rows [c_j ; k_rot_j] (D = R + rot)
// with its own latent query q' = [W_uk,h^T q_nope ; q_rot], and sums the SAME rows c_j.  So the
// heads (and neighbouring tokens of one sequence) are the 16 "query rows" of an MFMA tile and a
// cached row is loaded once for all of them.  One wave per (row group, key split):
//   S^T = K . Q'^T   A = cache rows straight from memory (lane: key l & 15, 8 contiguous d),
//                    B = Q'^T in registers (lane: query row l & 15, 8 contiguous d); a lane then
//                    holds 4 keys x 2 key tiles of ONE query row, so the softmax statistics of
//                    a row live in the lanes l, l ^ 16, l ^ 32, l ^ 48;
//   O^T += C^T . P^T A = the key-interleaved copy of c (groups of 4 keys contiguous per latent
//                    coordinate: 8 bytes per lane), B = P^T straight from the S^T accumulators,
//                    k slots 0-3 = keys 4g + j of tile 0, 4-7 = keys 4g + j of tile 1, as hi + lo
//                    bf16 parts (16 mantissa bits of each fp32 probability).
// No LDS and no barrier; scores, running max / sum and the output stay fp32.  Splits over the
// keys write (max, sum, unnormalised output) partials that latent_combine_kernel merges, so a
// single decoded token still fills the chip.
#include "k_layered.hpp"

namespace qie {
namespace lay {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ const uint16_t* page_base(const LatentCache& c, int slot, int pos, int64_t layer_off) {
    const int page = c.table[(int64_t)slot * c.max_pages + pos / c.page_tokens];
    return (const uint16_t*)c.pool + (int64_t)page * c.page_stride + layer_off;
}

template <int RT, int KS>
__global__ __launch_bounds__(64) void latent_attn_mfma_kernel(LatentAttnMfmaP p) {
    const int lane = threadIdx.x, g = lane >> 4, n = lane & 15;
    const int unit = blockIdx.x, grp = unit / p.S, sp = unit % p.S;
    const int4 G = p.groups[grp];   // first packed row, tokens, first head, heads per token
    const int nrows = G.y * G.w;
    const bool vrow = n < nrows;
    const int tok = G.x + (vrow ? n / G.w : 0), head = G.z + (vrow ? n % G.w : 0);
    const int slot = p.row_slot[G.x];
    const int mypos = p.row_pos[tok];
    const int hi = p.row_pos[G.x + G.y - 1];
    int lo = p.row_pos[G.x] - p.window + 1;
    if (lo < 0) lo = 0;
    const int R = p.R, D = p.R + p.rot, PT = p.cache.page_tokens;
    const int nrt = R >> 4;

    // this lane's query row as B fragments (bf16), zero beyond D and for unused rows
    bf16x8_t qf[KS];
    {
        const float* qa = p.q_abs + ((int64_t)tok * p.heads + head) * R;
        const float* qr = p.proj + (int64_t)tok * p.ld + (int64_t)head * (p.dim + p.rot) + p.dim;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int d0 = ks * 32 + 8 * g;
            uint32_t w[4] = {0u, 0u, 0u, 0u};
            if (vrow && d0 < D) {
                const float* src = d0 < R ? qa + d0 : qr + (d0 - R);   // R and rot are multiples of 8
#pragma unroll
                for (int j = 0; j < 4; j++) w[j] = pack2(src[2 * j], src[2 * j + 1]);
            }
            qf[ks] = __builtin_bit_cast(bf16x8_t, make_uint4(w[0], w[1], w[2], w[3]));
        }
    }

    const int kb_lo = lo >> 5, kb_hi = hi >> 5;
    const int per = (kb_hi - kb_lo + 1 + p.S - 1) / p.S;
    const int b0 = kb_lo + sp * per;
    int b1 = b0 + per;
    if (b1 > kb_hi + 1) b1 = kb_hi + 1;

    f32x4_t oacc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) oacc[rt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    for (int kb = b0; kb < b1; kb++) {
        const int k0 = kb << 5;
        f32x4_t sacc[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            sacc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            int key = k0 + 16 * t + n;
            if (key > hi) key = hi;   // masked below; keeps the address inside the slot's pages
            const uint16_t* row = page_base(p.cache, slot, key, p.layer_off) + (int64_t)(key % PT) * D;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                const int d0 = ks * 32 + 8 * g;
                uint4 kv = make_uint4(0u, 0u, 0u, 0u);
                if (d0 < D) kv = *reinterpret_cast<const uint4*>(row + d0);
                sacc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kv), qf[ks], sacc[t], 0, 0, 0);
            }
        }
        // scores of query row n against keys k0 + 16 t + 4 g + j
        float sv[8];
        float mloc = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int key = k0 + 16 * t + 4 * g + j;
                const bool ok = vrow && key <= mypos && key > mypos - p.window;
                const float s = ok ? sacc[t][j] * p.scale : -INFINITY;
                sv[4 * t + j] = s;
                mloc = fmaxf(mloc, s);
            }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
        const float m_new = fmaxf(m_run, mloc);
        float alpha = 1.f, pe[8];
        if (m_new == -INFINITY) {
#pragma unroll
            for (int i = 0; i < 8; i++) pe[i] = 0.f;
        } else {
            alpha = expf(m_run - m_new);
            float ls = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                pe[i] = expf(sv[i] - m_new);
                ls += pe[i];
            }
            l_run = l_run * alpha + ls;
            m_run = m_new;
        }
        // P = hi + lo bf16 parts, in k-slot order
        uint32_t ph[4], pl[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            ph[j] = pack2(pe[2 * j], pe[2 * j + 1]);
            pl[j] = pack2(pe[2 * j] - bf_lo(ph[j]), pe[2 * j + 1] - bf_hi(ph[j]));
        }
        const bf16x8_t pbh = __builtin_bit_cast(bf16x8_t, make_uint4(ph[0], ph[1], ph[2], ph[3]));
        const bf16x8_t pbl = __builtin_bit_cast(bf16x8_t, make_uint4(pl[0], pl[1], pl[2], pl[3]));
        // key-interleaved c: element ((key % PT) / 4 * R + r) * 4 + key % 4 after the PT x D rows
        const uint16_t* ct[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            int key4 = k0 + 16 * t + 4 * g;
            if (key4 > hi) key4 = hi & ~3;
            ct[t] = page_base(p.cache, slot, key4, p.layer_off) + (int64_t)PT * D + (int64_t)((key4 % PT) >> 2) * R * 4;
        }
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            if (rt < nrt) {
                const int r = 16 * rt + n;
                const uint2 v0 = *reinterpret_cast<const uint2*>(ct[0] + r * 4);
                const uint2 v1 = *reinterpret_cast<const uint2*>(ct[1] + r * 4);
                const bf16x8_t vf = __builtin_bit_cast(bf16x8_t, make_uint4(v0.x, v0.y, v1.x, v1.y));
                oacc[rt] = oacc[rt] * alpha;
                oacc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pbh, oacc[rt], 0, 0, 0);
                oacc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pbl, oacc[rt], 0, 0, 0);
            }
        }
    }
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (g == 0) {
        p.part_ml[((int64_t)unit * 16 + n) * 2] = m_run;
        p.part_ml[((int64_t)unit * 16 + n) * 2 + 1] = l_run;
    }
    float* po = p.part_o + ((int64_t)unit * 16 + n) * R;
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
        if (rt < nrt) *reinterpret_cast<float4*>(po + 16 * rt + 4 * g) = make_float4(oacc[rt][0], oacc[rt][1], oacc[rt][2], oacc[rt][3]);
}

// merges the key splits of one row group: out[tok, head, :] = sum_s e^(m_s - M) O_s / sum_s e^(m_s - M) l_s
__global__ __launch_bounds__(256) void latent_combine_kernel(LatentAttnMfmaP p) {
    const int grp = blockIdx.x;
    const int4 G = p.groups[grp];
    const int nrows = G.y * G.w, R = p.R;
    for (int n = 0; n < nrows; n++) {
        const int tok = G.x + n / G.w, head = G.z + n % G.w;
        float M = -INFINITY;
        for (int s = 0; s < p.S; s++) M = fmaxf(M, p.part_ml[(((int64_t)grp * p.S + s) * 16 + n) * 2]);
        float L = 0.f;
        for (int s = 0; s < p.S; s++) {
            const float* ml = p.part_ml + (((int64_t)grp * p.S + s) * 16 + n) * 2;
            if (ml[0] != -INFINITY) L += expf(ml[0] - M) * ml[1];
        }
        const float inv = 1.0f / L;
        float* o = p.out + ((int64_t)tok * p.heads + head) * R;
        for (int r = threadIdx.x; r < R; r += 256) {
            float acc = 0.f;
            for (int s = 0; s < p.S; s++) {
                const int64_t u = ((int64_t)grp * p.S + s) * 16 + n;
                const float m = p.part_ml[u * 2];
                if (m != -INFINITY) acc += expf(m - M) * p.part_o[u * R + r];
            }
            o[r] = acc * inv;
        }
    }
}

bool latent_attention_mfma_fits(int R, int rot) {
    return R % 16 == 0 && rot % 8 == 0 && R <= 512 && R + rot <= 576;
}

int latent_attention_mfma(const LatentAttnMfmaP& p, hipStream_t st) {
    QIE_REQUIRE(latent_attention_mfma_fits(p.R, p.rot), "latent attention (MFMA): latent %d + rotated %d not covered", p.R, p.rot);
    QIE_REQUIRE(p.n_groups > 0 && p.S > 0 && p.groups && p.part_o && p.part_ml, "latent attention (MFMA): bad arguments");
    QIE_REQUIRE(p.cache.page_tokens % 16 == 0, "latent attention (MFMA): pages of %d tokens", p.cache.page_tokens);
    const dim3 grid((unsigned)(p.n_groups * p.S)), block(64);
    const int D = p.R + p.rot;
    if (p.R <= 128 && D <= 160)
        hipLaunchKernelGGL((latent_attn_mfma_kernel<8, 5>), grid, block, 0, st, p);
    else if (p.R <= 256 && D <= 320)
        hipLaunchKernelGGL((latent_attn_mfma_kernel<16, 10>), grid, block, 0, st, p);
    else
        hipLaunchKernelGGL((latent_attn_mfma_kernel<32, 18>), grid, block, 0, st, p);
    QIE_LAUNCH_CHECK();
    hipLaunchKernelGGL(latent_combine_kernel, dim3(p.n_groups), dim3(256), 0, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

}  // namespace lay
}  // namespace qie
