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

// QG row groups per wave (consecutive groups of one entry: neighbouring tokens, or the head
// groups of one token) share every loaded cache fragment; the 4 waves of a workgroup take
// neighbouring units of the same key split, so their loads of the same rows meet in the L1.
template <int RT, int KS, int QG, int MINB>
__global__ __launch_bounds__(256, MINB) void latent_attn_mfma_kernel(LatentAttnMfmaP p) {
    const int lane = threadIdx.x & 63, g = lane >> 4, n = lane & 15;
    const int n_units = p.n_groups / QG;
    const int v = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (v >= n_units * p.S) return;
    const int sp = v / n_units, unit = v % n_units;
    const int R = p.R, D = p.R + p.rot, PT = p.cache.page_tokens;
    const int nrt = R >> 4;

    bool vrow[QG];
    int mypos[QG];
    bf16x8_t qf[QG][KS];
    int lo = 0x7fffffff, hi = -1, slot = 0, nq = 0;
#pragma unroll
    for (int q = 0; q < QG; q++) {
        const int4 G = p.groups[unit * QG + q];   // first packed row, tokens, first head, heads per token
        vrow[q] = n < G.y * G.w;
        const int tok = G.x + (vrow[q] ? n / G.w : 0), head = G.z + (vrow[q] ? n % G.w : 0);
        mypos[q] = p.row_pos[tok];
        if (G.y > 0) {
            nq = q + 1;
            slot = p.row_slot[G.x];
            lo = min(lo, p.row_pos[G.x]);
            hi = max(hi, p.row_pos[G.x + G.y - 1]);
        }
        // this lane's query row as B fragments (bf16), zero beyond D and for unused rows
        const float* qa = p.q_abs + ((int64_t)tok * p.heads + head) * R;
        const float* qr = p.proj + (int64_t)tok * p.ld + (int64_t)head * (p.dim + p.rot) + p.dim;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int d0 = ks * 32 + 8 * g;
            uint32_t w[4] = {0u, 0u, 0u, 0u};
            if (vrow[q] && d0 < D) {
                const float* src = d0 < R ? qa + d0 : qr + (d0 - R);   // R and rot are multiples of 8
#pragma unroll
                for (int j = 0; j < 4; j++) w[j] = pack2(src[2 * j], src[2 * j + 1]);
            }
            qf[q][ks] = __builtin_bit_cast(bf16x8_t, make_uint4(w[0], w[1], w[2], w[3]));
        }
    }
    lo = lo - p.window + 1;
    if (lo < 0) lo = 0;

    const int kb_lo = lo >> 5, kb_hi = hi >> 5;
    const int per = (kb_hi - kb_lo + 1 + p.S - 1) / p.S;
    const int b0 = kb_lo + sp * per;
    int b1 = b0 + per;
    if (b1 > kb_hi + 1) b1 = kb_hi + 1;

    f32x4_t oacc[QG][RT];
    float m_run[QG], l_run[QG];
#pragma unroll
    for (int q = 0; q < QG; q++) {
        m_run[q] = -INFINITY;
        l_run[q] = 0.f;
#pragma unroll
        for (int rt = 0; rt < RT; rt++) oacc[q][rt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    // page ids of the two 16-key tiles of a block (a tile never straddles a page), looked up one
    // block ahead so that no cache row load waits for a table load; keys past `hi` read row `hi`
    const int32_t* trow = p.cache.table + (int64_t)slot * p.cache.max_pages;
    const uint16_t* pool = (const uint16_t*)p.cache.pool + p.layer_off;
    const int pg_hi = hi >= 0 ? trow[hi / PT] : 0;
    int pgn[2];
#pragma unroll
    for (int t = 0; t < 2; t++) pgn[t] = b0 < b1 ? trow[min((b0 << 5) + 16 * t, hi) / PT] : 0;
    for (int kb = b0; kb < b1; kb++) {
        const int k0 = kb << 5;
        int pg[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            pg[t] = pgn[t];
            pgn[t] = trow[min(k0 + 32 + 16 * t, hi) / PT];
        }
        f32x4_t sacc[QG][2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
#pragma unroll
            for (int q = 0; q < QG; q++) sacc[q][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            int key = k0 + 16 * t + n;
            const bool past = key > hi;   // masked below; keeps the address inside the slot's pages
            if (past) key = hi;
            const uint16_t* row = pool + (int64_t)(past ? pg_hi : pg[t]) * p.cache.page_stride + (int64_t)(key % PT) * D;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                const int d0 = ks * 32 + 8 * g;
                // no branch around a load: loads inside conditional blocks are waited for one
                // by one; beyond D the query fragment is zero, so any finite values do
                const uint4 kv = *reinterpret_cast<const uint4*>(row + (d0 < D ? d0 : 0));
#pragma unroll
                for (int q = 0; q < QG; q++)
                    sacc[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kv), qf[q][ks], sacc[q][t],
                                                                         0, 0, 0);
            }
        }
        bf16x8_t pbh[QG], pbl[QG];
        float alpha[QG];
#pragma unroll
        for (int q = 0; q < QG; q++) {
            // scores of query row n against keys k0 + 16 t + 4 g + j
            float sv[8];
            float mloc = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int key = k0 + 16 * t + 4 * g + j;
                    const bool ok = vrow[q] && key <= mypos[q] && key > mypos[q] - p.window;
                    const float sc = ok ? sacc[q][t][j] * p.scale : -INFINITY;
                    sv[4 * t + j] = sc;
                    mloc = fmaxf(mloc, sc);
                }
            mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
            const float m_new = fmaxf(m_run[q], mloc);
            // branch-free (a branch here would fence the value loads below): while every key so
            // far is masked the reference max is 0, all weights and the rescale factor are 0
            float pe[8];
            const float m_ref = m_new == -INFINITY ? 0.f : m_new;
            alpha[q] = expf(m_run[q] - m_ref);
            float ls = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                pe[i] = expf(sv[i] - m_ref);
                ls += pe[i];
            }
            l_run[q] = l_run[q] * alpha[q] + ls;
            m_run[q] = m_new;
            // P = hi + lo bf16 parts, in k-slot order
            uint32_t ph[4], pl[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                ph[j] = pack2(pe[2 * j], pe[2 * j + 1]);
                pl[j] = pack2(pe[2 * j] - bf_lo(ph[j]), pe[2 * j + 1] - bf_hi(ph[j]));
            }
            pbh[q] = __builtin_bit_cast(bf16x8_t, make_uint4(ph[0], ph[1], ph[2], ph[3]));
            pbl[q] = __builtin_bit_cast(bf16x8_t, make_uint4(pl[0], pl[1], pl[2], pl[3]));
        }
        // key-interleaved c: element ((key % PT) / 4 * R + r) * 4 + key % 4 after the PT x D rows
        const uint16_t* ct[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            int key4 = k0 + 16 * t + 4 * g;
            const bool past = key4 > hi;
            if (past) key4 = hi & ~3;
            ct[t] = pool + (int64_t)(past ? pg_hi : pg[t]) * p.cache.page_stride + (int64_t)PT * D +
                    (int64_t)((key4 % PT) >> 2) * R * 4;
        }
        // Value product.  A latent size that fills the instantiation (the usual case) runs all
        // tiles with no branch in between, so the loads of the whole block are in flight together;
        // otherwise runs of 4 tiles behind one uniform branch each (a tile past R reads tile 0
        // again and its product is dropped at the end).
        auto pv_run = [&](const int rc, const int cnt) {
            uint2 v0[4], v1[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int r = (rc + i < cnt ? 16 * (rc + i) : 0) + n;
                v0[i] = *reinterpret_cast<const uint2*>(ct[0] + r * 4);
                v1[i] = *reinterpret_cast<const uint2*>(ct[1] + r * 4);
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const bf16x8_t vf = __builtin_bit_cast(bf16x8_t, make_uint4(v0[i].x, v0[i].y, v1[i].x, v1[i].y));
#pragma unroll
                for (int q = 0; q < QG; q++) {
                    oacc[q][rc + i] = oacc[q][rc + i] * alpha[q];
                    oacc[q][rc + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pbh[q], oacc[q][rc + i], 0, 0, 0);
                    oacc[q][rc + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pbl[q], oacc[q][rc + i], 0, 0, 0);
                }
            }
        };
        if (nrt == RT) {
#pragma unroll
            for (int rc = 0; rc < RT; rc += 4) pv_run(rc, RT);
        } else {
#pragma unroll
            for (int rc = 0; rc < RT; rc += 4)
                if (rc < nrt) pv_run(rc, nrt);
        }
    }
#pragma unroll
    for (int q = 0; q < QG; q++) {
        float l = l_run[q];
        l += __shfl_xor(l, 16, 64);
        l += __shfl_xor(l, 32, 64);
        const int64_t u = (((int64_t)(unit * QG + q)) * p.S + sp) * 16 + n;
        if (g == 0) {
            p.part_ml[u * 2] = m_run[q];
            p.part_ml[u * 2 + 1] = l;
        }
        float* po = p.part_o + u * R;
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
            if (rt < nrt)
                *reinterpret_cast<float4*>(po + 16 * rt + 4 * g) =
                    make_float4(oacc[q][rt][0], oacc[q][rt][1], oacc[q][rt][2], oacc[q][rt][3]);
    }
}

// merges the key splits of one (token, head) row: out = sum_s e^(m_s - M) O_s / sum_s e^(m_s - M) l_s.
// One block per row of a group; the split weights go through LDS so that the loads of the
// partial outputs are independent of each other.
__global__ __launch_bounds__(256) void latent_combine_kernel(LatentAttnMfmaP p) {
    __shared__ float w[64];
    __shared__ float inv_s;
    const int grp = blockIdx.x >> 4, n = blockIdx.x & 15;
    const int4 G = p.groups[grp];
    if (n >= G.y * G.w) return;
    const int tok = G.x + n / G.w, head = G.z + n % G.w, R = p.R, S = p.S;
    const int64_t u0 = (int64_t)grp * S * 16 + n;   // unit (grp, s) row n = u0 + 16 s
    if (threadIdx.x < 64) {
        const int s = threadIdx.x;
        const float m = s < S ? p.part_ml[(u0 + 16 * s) * 2] : -INFINITY;
        const float l = s < S ? p.part_ml[(u0 + 16 * s) * 2 + 1] : 0.f;
        float M = m;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o, 64));
        const float e = m == -INFINITY ? 0.f : expf(m - M);
        float L = e * l;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) L += __shfl_xor(L, o, 64);
        w[s] = e;
        if (s == 0) inv_s = 1.0f / L;
    }
    __syncthreads();
    const float inv = inv_s;
    float* o = p.out + ((int64_t)tok * p.heads + head) * R;
    for (int r = threadIdx.x; r < R; r += 256) {
        float acc = 0.f;
        for (int s = 0; s < S; s++) acc = fmaf(w[s], p.part_o[(u0 + 16 * s) * R + r], acc);
        o[r] = acc * inv;
    }
}

bool latent_attention_mfma_fits(int R, int rot) {
    return R % 16 == 0 && rot % 8 == 0 && R <= 512 && R + rot <= 576;
}

int latent_attention_mfma(const LatentAttnMfmaP& p, hipStream_t st) {
    QIE_REQUIRE(latent_attention_mfma_fits(p.R, p.rot), "latent attention (MFMA): latent %d + rotated %d not covered", p.R, p.rot);
    QIE_REQUIRE(p.n_groups > 0 && p.S > 0 && p.S <= 64 && p.groups && p.part_o && p.part_ml, "latent attention (MFMA): bad arguments");
    QIE_REQUIRE(p.cache.page_tokens % 16 == 0, "latent attention (MFMA): pages of %d tokens", p.cache.page_tokens);
    QIE_REQUIRE(p.n_groups % kLatentQG == 0, "latent attention (MFMA): %d groups are not whole units of %d", p.n_groups, kLatentQG);
    const int D = p.R + p.rot;
    const int waves = p.n_groups / kLatentQG * p.S;
    const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
    if (p.R <= 128 && D <= 160)
        hipLaunchKernelGGL((latent_attn_mfma_kernel<8, 5, kLatentQG, 2>), grid, block, 0, st, p);
    else if (p.R <= 256 && D <= 320)
        hipLaunchKernelGGL((latent_attn_mfma_kernel<16, 10, kLatentQG, 2>), grid, block, 0, st, p);
    else
        hipLaunchKernelGGL((latent_attn_mfma_kernel<32, 18, kLatentQG, 1>), grid, block, 0, st, p);
    QIE_LAUNCH_CHECK();
    hipLaunchKernelGGL(latent_combine_kernel, dim3(p.n_groups * 16), dim3(256), 0, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

}  // namespace lay
}  // namespace qie
