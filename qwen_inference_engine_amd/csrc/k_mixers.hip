// k_mixers.hip — mixers of the layered engine tier beside the latent attention (k_layered.hpp):
//
//   lay::gqa_post        q / k head norms, rotary (either pairing, partial), values turned by
//                        their position or taken from the raw keys, paged K / V append
//   lay::gqa_attention   grouped-query softmax attention over the paged rows with a causal,
//                        sliding or block-local mask and an optional log-distance bias; the
//                        weighted sum of turned values is turned back
//   lay::gated_scan      gated linear recurrence with an fp32 state per slot and head
//   lay::head_norm_rows  per-head RMS norm with a weight
//   lay::add_norm        residual add of a normed branch fused with the next branch's input norm
//
// Scores, softmax statistics, norms, gates and the recurrent state are fp32; cache rows are
// fp32 or bf16 by the engine's compute type.  A row's result depends only on its own slot,
// position and cache rows, never on what else the launch holds.
#include "k_layered.hpp"

namespace qie {
namespace lay {

namespace {

template <typename T> __device__ __forceinline__ float ldc(const T* p, int64_t i);
template <> __device__ __forceinline__ float ldc<float>(const float* p, int64_t i) { return p[i]; }
template <> __device__ __forceinline__ float ldc<uint16_t>(const uint16_t* p, int64_t i) { return bf2f(p[i]); }
template <typename T> __device__ __forceinline__ void stc(T* p, int64_t i, float v);
template <> __device__ __forceinline__ void stc<float>(float* p, int64_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void stc<uint16_t>(uint16_t* p, int64_t i, float v) { p[i] = f2bf(v); }

__device__ __forceinline__ float wsum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wmax(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float bsum256(float v, float* red) {
    v = wsum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// Coordinate i of `buf` after the turn by the angles whose cos / sin are cs / sn (one per pair);
// only the first `dims` coordinates turn.  The pair (u, w) becomes (u c - w s, w c + u s);
// sign = -1 turns back.
__device__ __forceinline__ float turned(const float* buf, int i, int dims, int layout, const float* cs, const float* sn, float sign) {
    if (i >= dims) return buf[i];
    int j, partner;
    float sg;
    if (layout == 1) {
        j = i >> 1;
        partner = i ^ 1;
        sg = (i & 1) ? 1.f : -1.f;
    } else {
        const int half = dims >> 1;
        if (i < half) {
            j = i;
            partner = i + half;
            sg = -1.f;
        } else {
            j = i - half;
            partner = j;
            sg = 1.f;
        }
    }
    return buf[i] * cs[j] + sg * sign * buf[partner] * sn[j];
}

__device__ __forceinline__ int64_t page_base(const LatentCache& c, int slot, int pos) {
    const int page = c.table[(int64_t)slot * c.max_pages + pos / c.page_tokens];
    return (int64_t)page * c.page_stride;
}

}  // namespace

// ------------------------------------------------------------------ post-projection
// One block per row; a wave per head, the head's coordinates staged in LDS so that either pairing
// finds its partner.
template <typename TC>
__global__ __launch_bounds__(256) void gqa_post_kernel(GqaPostP p) {
    extern __shared__ float sm[];
    const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int slot = p.row_slot[t], pos = p.row_pos[t];
    const int mx = max(p.dim, p.vdim);
    float* buf = sm + wave * mx;
    float* row = p.proj + (int64_t)t * p.ld;
    const int64_t pb = page_base(p.cache, slot, pos);
    const int pt = pos % p.cache.page_tokens;
    const int H = p.heads, G = p.kv_heads, dim = p.dim, vdim = p.vdim;
    TC* krow = (TC*)p.cache.pool + pb + p.k_off + (int64_t)pt * G * dim;
    TC* vrow = (TC*)p.cache.pool + pb + p.v_off + (int64_t)pt * G * vdim;
    const float* cs = p.rope_cos + (int64_t)pos * (p.rot_dims / 2);
    const float* sn = p.rope_sin + (int64_t)pos * (p.rot_dims / 2);
    for (int h0 = 0; h0 < H + G; h0 += 4) {
        const int hh = h0 + wave;
        const bool on = hh < H + G, is_q = hh < H;
        float* x = row + (is_q ? p.q_col + hh * dim : p.k_col + (hh - H) * dim);
        if (on) {
            float ss = 0.f;
            for (int i = lane; i < dim; i += 64) {
                const float a = x[i];
                buf[i] = a;
                ss += a * a;
            }
            ss = wsum(ss);
            if (!is_q && p.v_col < 0)   // the value is the key as projected
                for (int i = lane; i < dim; i += 64) stc<TC>(vrow, (int64_t)(hh - H) * dim + i, buf[i]);
            if (p.qk_norm) {
                const float inv = 1.0f / sqrtf(ss / (float)dim + p.eps);
                const float* w = p.qk_norm == 1 ? (is_q ? p.qn_w : p.kn_w) : nullptr;
                for (int i = lane; i < dim; i += 64) buf[i] = buf[i] * inv * (w ? w[i] : 1.0f);
            }
        }
        __syncthreads();
        if (on)
            for (int i = lane; i < dim; i += 64) {
                const float o = turned(buf, i, p.rot_dims, p.rot_layout, cs, sn, 1.f);
                if (is_q)
                    x[i] = o;
                else
                    stc<TC>(krow, (int64_t)(hh - H) * dim + i, o);
            }
        __syncthreads();
    }
    if (p.v_col < 0) return;
    const float* vcs = p.rot_values ? p.vrope_cos + (int64_t)pos * (vdim / 2) : nullptr;
    const float* vsn = p.rot_values ? p.vrope_sin + (int64_t)pos * (vdim / 2) : nullptr;
    for (int g0 = 0; g0 < G; g0 += 4) {
        const int g = g0 + wave;
        const bool on = g < G;
        if (on)
            for (int i = lane; i < vdim; i += 64) buf[i] = row[p.v_col + g * vdim + i];
        __syncthreads();
        if (on)
            for (int i = lane; i < vdim; i += 64)
                stc<TC>(vrow, (int64_t)g * vdim + i, p.rot_values ? turned(buf, i, vdim, p.rot_layout, vcs, vsn, 1.f) : buf[i]);
        __syncthreads();
    }
}

int gqa_post(const GqaPostP& p, bool cache_f32, int T, hipStream_t st) {
    QIE_REQUIRE(p.heads > 0 && p.kv_heads > 0 && p.heads % p.kv_heads == 0, "gqa_post: %d query heads over %d key heads", p.heads,
                p.kv_heads);
    QIE_REQUIRE(p.rot_dims % 2 == 0 && p.rot_dims <= p.dim, "gqa_post: rotary dims %d must be even and <= %d", p.rot_dims, p.dim);
    QIE_REQUIRE(!p.rot_values || p.vdim % 2 == 0, "gqa_post: turned values need an even vdim (%d)", p.vdim);
    QIE_REQUIRE(p.v_col >= 0 || p.vdim == p.dim, "gqa_post: keys as values need vdim == dim");
    const size_t shm = (size_t)4 * std::max(p.dim, p.vdim) * 4;
    QIE_REQUIRE(shm <= 48 * 1024, "gqa_post: head size %d above the kernel's staging", std::max(p.dim, p.vdim));
    if (cache_f32)
        hipLaunchKernelGGL(gqa_post_kernel<float>, dim3(T), dim3(256), shm, st, p);
    else
        hipLaunchKernelGGL(gqa_post_kernel<uint16_t>, dim3(T), dim3(256), shm, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ attention, exact form
// One block per (head, row): the visible keys go through in chunks of GA_CHUNK with a running
// maximum and sum; a wave scores a key, a thread owns value coordinates.
constexpr int GA_CHUNK = 256;
constexpr int GA_MAXV = 4;   // vdim <= 256 * GA_MAXV

__device__ __forceinline__ int first_visible(int mask, int size, int pos) {
    if (mask == 1) return max(0, pos - size + 1);
    if (mask == 2) return pos / size * size;
    return 0;
}

template <typename TC>
__global__ __launch_bounds__(256) void gqa_attention_kernel(GqaAttnP p) {
    extern __shared__ float sm[];
    float* q = sm;                 // [dim]
    float* sc = sm + p.dim;        // [GA_CHUNK]
    float* ob = sc + GA_CHUNK;     // [vdim]
    __shared__ float red[4];
    const int h = blockIdx.x, t = blockIdx.y, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int slot = p.row_slot[t], pos = p.row_pos[t];
    const int dim = p.dim, vdim = p.vdim, G = p.kv_heads, g = h / (p.heads / G);
    const float* qr = p.proj + (int64_t)t * p.ld + p.q_col + h * dim;
    for (int i = tid; i < dim; i += 256) q[i] = qr[i];
    __syncthreads();
    const int lo = first_visible(p.mask, p.mask_size, pos);
    const float b1 = p.r1 ? p.r1[h] : 0.f, b2 = p.r1 ? p.r2[h] : 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    float acc[GA_MAXV] = {};
    for (int j0 = lo; j0 <= pos; j0 += GA_CHUNK) {
        const int nk = min(GA_CHUNK, pos + 1 - j0);
        for (int jj = wave; jj < nk; jj += 4) {
            const int j = j0 + jj;
            const TC* k = (const TC*)p.cache.pool + page_base(p.cache, slot, j) + p.k_off +
                          ((int64_t)(j % p.cache.page_tokens) * G + g) * dim;
            float s = 0.f;
            for (int i = lane; i < dim; i += 64) s = fmaf(q[i], ldc<TC>(k, i), s);
            s = wsum(s);
            if (lane == 0) {
                s *= p.scale;
                if (p.r1) s -= b1 * log1pf(b2 * (float)(pos - j));
                sc[jj] = s;
            }
        }
        __syncthreads();
        float mx = -INFINITY;
        for (int jj = tid; jj < nk; jj += 256) mx = fmaxf(mx, sc[jj]);
        mx = wmax(mx);
        if (lane == 0) red[wave] = mx;
        __syncthreads();
        mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        const float m_new = fmaxf(m_run, mx);
        const float alpha = expf(m_run - m_new);   // 0 on the first chunk
        __syncthreads();
        float ls = 0.f;
        for (int jj = tid; jj < nk; jj += 256) {
            const float e = expf(sc[jj] - m_new);
            sc[jj] = e;
            ls += e;
        }
        ls = bsum256(ls, red);
        l_run = l_run * alpha + ls;
        m_run = m_new;
#pragma unroll
        for (int i = 0; i < GA_MAXV; i++) acc[i] *= alpha;
        for (int jj = 0; jj < nk; jj++) {
            const int j = j0 + jj;
            const TC* v = (const TC*)p.cache.pool + page_base(p.cache, slot, j) + p.v_off +
                          ((int64_t)(j % p.cache.page_tokens) * G + g) * vdim;
            const float w = sc[jj];
#pragma unroll
            for (int i = 0; i < GA_MAXV; i++) {
                const int r = tid + i * 256;
                if (r < vdim) acc[i] = fmaf(w, ldc<TC>(v, r), acc[i]);
            }
        }
        __syncthreads();
    }
    const float inv = 1.0f / l_run;
#pragma unroll
    for (int i = 0; i < GA_MAXV; i++) {
        const int r = tid + i * 256;
        if (r < vdim) ob[r] = acc[i] * inv;
    }
    __syncthreads();
    const float* vcs = p.rot_values ? p.vrope_cos + (int64_t)pos * (vdim / 2) : nullptr;
    const float* vsn = p.rot_values ? p.vrope_sin + (int64_t)pos * (vdim / 2) : nullptr;
    const int64_t o0 = (int64_t)t * p.ld_out + p.out_col + (int64_t)h * vdim;
    for (int r = tid; r < vdim; r += 256) {
        const float o = (p.rot_values ? turned(ob, r, vdim, p.rot_layout, vcs, vsn, -1.f) : ob[r]) * p.out_scale;
        p.out[o0 + r] = o;
        if (p.out_bf) p.out_bf[o0 + r] = f2bf(o);
    }
}

int gqa_attention(const GqaAttnP& p, bool cache_f32, int T, hipStream_t st) {
    QIE_REQUIRE(p.vdim <= 256 * GA_MAXV, "gqa attention: vdim %d above %d", p.vdim, 256 * GA_MAXV);
    QIE_REQUIRE(p.mask == 0 || p.mask_size >= 1, "gqa attention: mask size %d", p.mask_size);
    QIE_REQUIRE(p.heads % p.kv_heads == 0, "gqa attention: %d query heads over %d key heads", p.heads, p.kv_heads);
    const size_t shm = (size_t)(p.dim + GA_CHUNK + p.vdim) * 4;
    QIE_REQUIRE(shm <= 48 * 1024, "gqa attention: head size above the kernel's staging");
    if (cache_f32)
        hipLaunchKernelGGL(gqa_attention_kernel<float>, dim3(p.heads, T), dim3(256), shm, st, p);
    else
        hipLaunchKernelGGL(gqa_attention_kernel<uint16_t>, dim3(p.heads, T), dim3(256), shm, st, p);
    QIE_LAUNCH_CHECK();
    return 0;
}

bool gqa_attention_mfma_fits(int dim, int vdim) { return false; }
int gqa_attention_mfma(const GqaAttnMfmaP& p, hipStream_t st) { return fail(-22, "gqa attention: no matrix-core form for these sizes"); }

// ------------------------------------------------------------------ gated linear recurrence
// One block per (head, entry, 64 value columns).  A thread owns one column of SR state rows in
// registers; blockDim / 64 thread groups split the dim rows.  The entry's rows go through in
// tiles: the tile's q, f (activations applied, fp32) and v are staged in LDS, every token then
// costs SR multiply-adds per thread with no synchronisation; the groups' partial outputs meet in
// LDS once a tile.  Rows beyond dim are padded with f = 1, q = 0 (their state stays 0).
constexpr int SR = 32;

__global__ __launch_bounds__(1024) void gated_scan_kernel(GatedScanP p, int TT, int dimP) {
    extern __shared__ float sm[];
    const int NG = blockDim.x >> 6;
    float* qs = sm;                       // [TT][dimP]
    float* fs = qs + TT * dimP;           // [TT][dimP]
    float* vs = fs + TT * dimP;           // [TT][64]
    float* op = vs + TT * 64;             // [TT][NG][64]
    const int h = blockIdx.x, c0 = blockIdx.z * 64, tid = threadIdx.x, lane = tid & 63, grp = tid >> 6;
    const int4 en = p.entries[blockIdx.y];
    const int dim = p.dim, vdim = p.vdim, c = c0 + lane, d0 = grp * SR;
    const bool cok = c < vdim;
    float* stp = p.state + (int64_t)en.z * p.slot_stride + p.state_off + (int64_t)h * dim * vdim;
    float S[SR];
#pragma unroll
    for (int r = 0; r < SR; r++) {
        const int d = d0 + r;
        S[r] = (en.w > 0 && d < dim && cok) ? stp[(int64_t)d * vdim + c] : 0.f;
    }
    const int64_t HV = (int64_t)p.heads * vdim;
    for (int t0 = 0; t0 < en.y; t0 += TT) {
        const int nt = min(TT, en.y - t0);
        __syncthreads();
        for (int i = tid; i < nt * dimP; i += blockDim.x) {
            const int tt = i / dimP, d = i % dimP;
            float qv = 0.f, fv = 1.f;
            if (d < dim) {
                const float* row = p.proj + (int64_t)(en.x + t0 + tt) * p.ld;
                const float zq = row[p.q_col + h * dim + d];
                qv = zq / (1.0f + expf(-zq));
                const float zf = row[p.f_col + h * dim + d] + p.f_bias[h * dim + d];
                const float l = p.lower[h * dim + d];
                fv = l + (1.0f - l) * (1.0f / (1.0f + expf(-zf)));
            }
            qs[i] = qv;
            fs[i] = fv;
        }
        for (int i = tid; i < nt * 64; i += blockDim.x) {
            const int tt = i >> 6, cc = c0 + (i & 63);
            vs[i] = cc < vdim ? p.proj[(int64_t)(en.x + t0 + tt) * p.ld + p.v_col + h * vdim + cc] : 0.f;
        }
        __syncthreads();
        for (int tt = 0; tt < nt; tt++) {
            const float v = vs[tt * 64 + lane];
            const float* ft = fs + tt * dimP + d0;
            const float* qt = qs + tt * dimP + d0;
            float o = 0.f;
#pragma unroll
            for (int r = 0; r < SR; r++) {
                const float f = ft[r];
                S[r] = fmaf(f, S[r], (1.0f - f) * v);
                o = fmaf(S[r], qt[r], o);
            }
            op[(tt * NG + grp) * 64 + lane] = o;
        }
        __syncthreads();
        for (int i = tid; i < nt * 64; i += blockDim.x) {
            const int tt = i >> 6, cl = i & 63;
            float o = 0.f;
            for (int gI = 0; gI < NG; gI++) o += op[(tt * NG + gI) * 64 + cl];
            if (c0 + cl < vdim) p.out[(int64_t)(en.x + t0 + tt) * HV + (int64_t)h * vdim + c0 + cl] = o;
        }
    }
#pragma unroll
    for (int r = 0; r < SR; r++) {
        const int d = d0 + r;
        if (d < dim && cok) stp[(int64_t)d * vdim + c] = S[r];
    }
}

int gated_scan(const GatedScanP& p, hipStream_t st) {
    QIE_REQUIRE(p.n_entries > 0 && p.heads > 0 && p.dim > 0 && p.vdim > 0, "gated scan: bad sizes");
    const int NG = (p.dim + SR - 1) / SR;
    QIE_REQUIRE(NG <= 16, "gated scan: dim %d above %d", p.dim, 16 * SR);
    const int dimP = NG * SR;
    const int per_tok = (2 * dimP + 64 + NG * 64) * 4;
    const int TT = std::max(1, std::min(16, 48 * 1024 / per_tok));
    const size_t shm = (size_t)TT * per_tok;
    dim3 grid((unsigned)p.heads, (unsigned)p.n_entries, (unsigned)((p.vdim + 63) / 64));
    hipLaunchKernelGGL(gated_scan_kernel, grid, dim3(64 * NG), shm, st, p, TT, dimP);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ per-head norm
__global__ __launch_bounds__(256) void head_norm_rows_kernel(const float* o, const float* w, float eps, float scale, int heads, int vdim,
                                                             float* out, uint16_t* out_bf, int64_t ld_out, int out_col) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int h = wave; h < heads; h += 4) {
        const float* x = o + (t * heads + h) * vdim;
        float ss = 0.f;
        for (int i = lane; i < vdim; i += 64) ss += x[i] * x[i];
        ss = wsum(ss);
        const float inv = scale / sqrtf(ss / (float)vdim + eps);
        const int64_t o0 = t * ld_out + out_col + (int64_t)h * vdim;
        for (int i = lane; i < vdim; i += 64) {
            const float y = x[i] * inv * w[i];
            out[o0 + i] = y;
            if (out_bf) out_bf[o0 + i] = f2bf(y);
        }
    }
}
int head_norm_rows(const float* o, const float* w, float eps, float scale, int heads, int vdim, int T, float* out, uint16_t* out_bf,
                   int64_t ld_out, int out_col, hipStream_t st) {
    hipLaunchKernelGGL(head_norm_rows_kernel, dim3(T), dim3(256), 0, st, o, w, eps, scale, heads, vdim, out, out_bf, ld_out, out_col);
    QIE_LAUNCH_CHECK();
    return 0;
}

// ------------------------------------------------------------------ residual add + next norm
__global__ __launch_bounds__(256) void add_norm_kernel(float* x, const float* xin, const float* v, const float* wb, const float* add,
                                                       const float* wn, float* h, uint16_t* h_bf, int W, float eps) {
    __shared__ float red[4];
    const int64_t r0 = (int64_t)blockIdx.x * W;
    float inv_v = 0.f;
    if (v) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < W; i += 256) {
            const float a = v[r0 + i];
            ss += a * a;
        }
        ss = bsum256(ss, red);
        inv_v = 1.0f / sqrtf(ss / (float)W + eps);
    }
    float sx = 0.f;
    for (int i = threadIdx.x; i < W; i += 256) {
        float a = xin[r0 + i];
        if (v) a += v[r0 + i] * inv_v * (1.0f + wb[i]);
        if (add) a += add[r0 + i];
        if (v || add || xin != x) x[r0 + i] = a;
        sx += a * a;
    }
    if (!wn) return;
    sx = bsum256(sx, red);
    const float inv_x = 1.0f / sqrtf(sx / (float)W + eps);
    for (int i = threadIdx.x; i < W; i += 256) {
        const float o = x[r0 + i] * inv_x * (1.0f + wn[i]);   // the thread's own store above
        h[r0 + i] = o;
        if (h_bf) h_bf[r0 + i] = f2bf(o);
    }
}
int add_norm(float* x, const float* xin, const float* v, const float* wb, const float* add, const float* wn, float* h, uint16_t* h_bf,
             int T, int W, float eps, hipStream_t st) {
    QIE_REQUIRE(x && xin && (!v || wb) && (!wn || h), "add_norm: bad arguments");
    hipLaunchKernelGGL(add_norm_kernel, dim3(T), dim3(256), 0, st, x, xin, v, wb, add, wn, h, h_bf, W, eps);
    QIE_LAUNCH_CHECK();
    return 0;
}

}  // namespace lay
}  // namespace qie
