// lm_mix.hip — the row-wise and sequence-wise kernels of the layered-model tier: embedding, RMS norms (with the token shift and
// the residual sum fused in), the gated linear recurrence (HGRN2) and the latent attention over a paged cache of latents.
// Everything here is fp32 in both precision modes: norms, gates, the recurrent state, positions, angles, scores and weights.
#include <math.h>

#include "lm_kernels.h"

namespace zg {
namespace lm {

namespace {

__device__ __forceinline__ float block_allsum(float v, float* s_red) {
    v = wave_allsum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) s_red[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < nw; ++w) t += s_red[w];
    return t;
}

// 1 / sqrt(mean(v^2) + eps) of one row, the same summation order wherever a row is normed (a row normed again as somebody's
// predecessor gives the bits its own workgroup got).
__device__ __forceinline__ float row_inv_rms(const float* v, int n, float eps, float* s_red) {
    float ss = 0.0f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) ss = fmaf(v[i], v[i], ss);
    ss = block_allsum(ss, s_red);
    return 1.0f / sqrtf(ss / (float)n + eps);
}

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

__global__ __launch_bounds__(256) void embed_kernel(const bf16_t* table, const int* ids, float* x, int W, int vocab, int* flag) {
    const int m = blockIdx.x, id = ids[m];
    const bool ok = id >= 0 && id < vocab;
    if (!ok && threadIdx.x == 0) *flag = 1;
    const bf16_t* row = table + (size_t)(ok ? id : 0) * W;
    for (int i = threadIdx.x; i < W; i += blockDim.x) x[(size_t)m * W + i] = ok ? __uint_as_float((uint32_t)row[i] << 16) : 0.0f;
}

__global__ __launch_bounds__(256) void norm_shift_kernel(const float* x, const float* w, const float* mu, float eps, float* out, int W,
                                                         const int* row_prev, const int* row_slot, const float* shift_state,
                                                         size_t slot_stride, const int* row_entry_if_last, float* last_out) {
    __shared__ float s_red[8];
    const int m = blockIdx.x;
    const float* xr = x + (size_t)m * W;
    const float r = row_inv_rms(xr, W, eps, s_red);
    const int entry = row_entry_if_last ? row_entry_if_last[m] : -1;
    if (mu == nullptr) {
        for (int i = threadIdx.x; i < W; i += blockDim.x) {
            const float h = xr[i] * r * (1.0f + w[i]);
            out[(size_t)m * W + i] = h;
            if (entry >= 0) last_out[(size_t)entry * W + i] = h;
        }
        return;
    }
    const int pm = row_prev[m];
    const float* xp = nullptr;
    const float* hp = nullptr;
    float rp = 0.0f;
    if (pm >= 0) {
        xp = x + (size_t)pm * W;
        rp = row_inv_rms(xp, W, eps, s_red);
    } else {
        hp = shift_state + (size_t)row_slot[m] * slot_stride;
    }
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
        const float g = 1.0f + w[i];
        const float h = xr[i] * r * g;
        const float before = xp ? xp[i] * rp * g : hp[i];
        out[(size_t)m * W + i] = h + (before - h) * mu[i];
        if (entry >= 0) last_out[(size_t)entry * W + i] = h;
    }
}

__global__ __launch_bounds__(256) void commit_rows_kernel(float* dst, size_t slot_stride, const float* src, size_t src_stride, const int* slots,
                                                          int width, size_t dst_set_stride, size_t src_set_stride) {
    const int e = blockIdx.x, set = blockIdx.y;
    float* d = dst + (size_t)slots[e] * slot_stride + set * dst_set_stride;
    const float* s = src + (size_t)e * src_stride + set * src_set_stride;
    for (int i = threadIdx.x; i < width; i += blockDim.x) d[i] = s[i];
}

__global__ __launch_bounds__(256) void norm_add_kernel(float* x, const float* y, const float* w, float eps, int W) {
    __shared__ float s_red[8];
    const int m = blockIdx.x;
    const float* yr = y + (size_t)m * W;
    const float r = row_inv_rms(yr, W, eps, s_red);
    for (int i = threadIdx.x; i < W; i += blockDim.x) x[(size_t)m * W + i] += yr[i] * r * (1.0f + w[i]);
}

__global__ __launch_bounds__(256) void norm_gather_kernel(const float* x, const int* rows, const float* w, float eps, float* out, int W) {
    __shared__ float s_red[8];
    const int j = blockIdx.x;
    const float* xr = x + (size_t)rows[j] * W;
    const float r = row_inv_rms(xr, W, eps, s_red);
    for (int i = threadIdx.x; i < W; i += blockDim.x) out[(size_t)j * W + i] = xr[i] * r * (1.0f + w[i]);
}

// one wave per (row, head) vector
__global__ __launch_bounds__(256) void norm_plain_kernel(float* v, int ld, int rows_per_m, int width, int n_vec, const float* w, float eps) {
    const int vec = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (vec >= n_vec) return;
    float* p = v + (size_t)(vec / rows_per_m) * ld + (size_t)(vec % rows_per_m) * width;
    float ss = 0.0f;
    for (int i = lane; i < width; i += 64) ss = fmaf(p[i], p[i], ss);
    ss = wave_allsum(ss);
    const float r = 1.0f / sqrtf(ss / (float)width + eps);
    for (int i = lane; i < width; i += 64) p[i] = p[i] * r * w[i];
}

// ------------------------------------------------------------------------------------------------ HGRN2
__global__ __launch_bounds__(256) void hgrn2_gates_kernel(float* proj, int ld, int M, int HD, const float* bias, const float* low) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)M * HD) return;
    const int m = (int)(idx / HD), i = (int)(idx % HD);
    float* row = proj + (size_t)m * ld;
    row[i] = silu_f(row[i]);
    const float l = low[i];
    row[HD + i] = l + (1.0f - l) * sigmoid_f(row[HD + i] + bias[i]);
}

// A column j of a head's state S[D][V] is held by G consecutive lanes, 16 rows each (D <= 16 G); the token loop is serial, the
// next token's gates are fetched while the current one is applied.
constexpr int kScanRows = 16;
template <int G>
__global__ __launch_bounds__(256) void hgrn2_scan_kernel(const float* proj, int ld, float* out, int ldo, float* state, size_t slot_stride,
                                                         const int* ent_start, const int* ent_len, const int* ent_slot, int H, int D, int V) {
    const int e = blockIdx.x, h = blockIdx.y;
    const int cols = blockDim.x / G;
    const int j = blockIdx.z * cols + threadIdx.x / G, g = threadIdx.x % G;
    const bool col_ok = j < V;
    const int HD = H * D, T = ent_len[e], m0 = ent_start[e];
    float* S_mem = state + (size_t)ent_slot[e] * slot_stride + (size_t)h * D * V;
    float S[kScanRows];
    bool ok[kScanRows];
#pragma unroll
    for (int r = 0; r < kScanRows; ++r) {
        const int i = g * kScanRows + r;
        ok[r] = col_ok && i < D;
        S[r] = ok[r] ? S_mem[(size_t)i * V + j] : 0.0f;
    }
    const int qoff = h * D + g * kScanRows, foff = HD + qoff, voff = 2 * HD + h * V + j;
    float q[kScanRows], f[kScanRows], v = 0.0f;
    auto fetch = [&](int t, float* qd, float* fd, float& vd) {
        const float* row = proj + (size_t)(m0 + t) * ld;
#pragma unroll
        for (int r = 0; r < kScanRows; ++r) {
            qd[r] = ok[r] ? row[qoff + r] : 0.0f;
            fd[r] = ok[r] ? row[foff + r] : 1.0f;
        }
        vd = col_ok ? row[voff] : 0.0f;
    };
    if (T > 0) fetch(0, q, f, v);
    for (int t = 0; t < T; ++t) {
        float qn[kScanRows], fn[kScanRows], vn = 0.0f;
        if (t + 1 < T) fetch(t + 1, qn, fn, vn);
        float o = 0.0f;
#pragma unroll
        for (int r = 0; r < kScanRows; ++r) {
            S[r] = fmaf(f[r], S[r], (1.0f - f[r]) * v);
            o = fmaf(S[r], q[r], o);
        }
#pragma unroll
        for (int off = 1; off < G; off <<= 1) o += __shfl_xor(o, off, 64);
        if (g == 0 && col_ok) out[(size_t)(m0 + t) * ldo + h * V + j] = o;
        if (t + 1 < T) {
#pragma unroll
            for (int r = 0; r < kScanRows; ++r) {
                q[r] = qn[r];
                f[r] = fn[r];
            }
            v = vn;
        }
    }
#pragma unroll
    for (int r = 0; r < kScanRows; ++r)
        if (ok[r]) S_mem[(size_t)(g * kScanRows + r) * V + j] = S[r];
}

// ------------------------------------------------------------------------------------------------ latent attention
__device__ __forceinline__ size_t cache_row(const int* page_table, int max_pages, int page_tokens, int slot, int pos) {
    return (size_t)page_table[(size_t)slot * max_pages + pos / page_tokens] * page_tokens + pos % page_tokens;
}

// the interleaved pair (2i, 2i + 1) of `src` at position pos, rotated by pos * freq[i]; angle and product in fp32
__device__ __forceinline__ void rotate_pair(const float* src, float* dst, int i, int pos, const Rotary& rot) {
    const float a = (float)pos * rot.freq[i];
    const float c = cosf(a) * rot.amp, s = sinf(a) * rot.amp;
    const float u = src[2 * i], v = src[2 * i + 1];
    dst[2 * i] = u * c - v * s;
    dst[2 * i + 1] = v * c + u * s;
}

__global__ __launch_bounds__(256) void latent_prep_kernel(const float* proj, int ld, int q_rank, int KR, int R, const float* wq, const float* wkv,
                                                          float eps, Rotary rot, const int* row_pos, const int* row_slot, const int* page_table,
                                                          int max_pages, int page_tokens, float* cq, float* cache) {
    __shared__ float s_red[8];
    const int m = blockIdx.x;
    const float* row = proj + (size_t)m * ld;
    const float rq = row_inv_rms(row, q_rank, eps, s_red);
    const float rc = row_inv_rms(row + q_rank, KR, eps, s_red);
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x) cq[(size_t)m * q_rank + i] = row[i] * rq * wq[i];
    const int pos = row_pos[m];
    float* crow = cache + cache_row(page_table, max_pages, page_tokens, row_slot[m], pos) * (size_t)(KR + R);
    for (int i = threadIdx.x; i < KR; i += blockDim.x) crow[i] = row[q_rank + i] * rc * wkv[i];
    const float* kr = row + q_rank + KR;
    for (int i = threadIdx.x; i < rot.dims / 2; i += blockDim.x) rotate_pair(kr, crow + KR, i, pos, rot);
    for (int i = rot.dims + threadIdx.x; i < R; i += blockDim.x) crow[KR + i] = kr[i];
}

__global__ __launch_bounds__(256) void q_rotary_kernel(const float* q, int ldq, float* qa, int ldqa, int H, int D, int R, int KR, Rotary rot,
                                                       const int* row_pos) {
    const int m = blockIdx.x, pos = row_pos[m], half = rot.dims / 2;
    for (int idx = threadIdx.x; idx < H * half; idx += blockDim.x) {
        const int h = idx / half, i = idx % half;
        rotate_pair(q + (size_t)m * ldq + (size_t)h * (D + R) + D, qa + (size_t)m * ldqa + (size_t)h * (KR + R) + KR, i, pos, rot);
    }
    const int rest = R - rot.dims;
    for (int idx = threadIdx.x; idx < H * rest; idx += blockDim.x) {
        const int h = idx / rest, i = rot.dims + idx % rest;
        qa[(size_t)m * ldqa + (size_t)h * (KR + R) + KR + i] = q[(size_t)m * ldq + (size_t)h * (D + R) + D + i];
    }
}

// One workgroup per (row, head).  The lanes of a wave split the KR + R dimensions of a cache row (ND per lane); a wave walks
// its share of the keys four at a time with a running (maximum, sum, weighted latent) and the four waves are merged at the end.
template <int ND>
__global__ __launch_bounds__(256) void latent_attention_kernel(const float* qa, float* ctx, int H, int KR, int R, float scale, const int* row_pos,
                                                               const int* row_slot, const int* page_table, int max_pages, int page_tokens,
                                                               const float* cache) {
    __shared__ float s_m[4], s_l[4];
    __shared__ float s_acc[4][ND * 64];
    const int m = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int DT = KR + R, n_keys = row_pos[m] + 1, slot = row_slot[m];
    const float* qrow = qa + ((size_t)m * H + h) * DT;
    float q[ND], acc[ND];
#pragma unroll
    for (int i = 0; i < ND; ++i) {
        const int d = lane + 64 * i;
        q[i] = d < DT ? qrow[d] : 0.0f;
        acc[i] = 0.0f;
    }
    float mx = -INFINITY, l = 0.0f;
    const int* pt = page_table + (size_t)slot * max_pages;
    for (int kb = wave * 4; kb < n_keys; kb += 16) {
        float r[4][ND], s[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int key = kb + u < n_keys ? kb + u : kb;
            const float* row = cache + ((size_t)pt[key / page_tokens] * page_tokens + key % page_tokens) * DT;
            float part = 0.0f;
#pragma unroll
            for (int i = 0; i < ND; ++i) {
                const int d = lane + 64 * i;
                r[u][i] = d < DT ? row[d] : 0.0f;
                part = fmaf(q[i], r[u][i], part);
            }
            s[u] = part;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            s[u] = wave_allsum(s[u]) * scale;
            if (kb + u >= n_keys) s[u] = -INFINITY;
        }
        const float mn = fmaxf(fmaxf(mx, s[0]), fmaxf(fmaxf(s[1], s[2]), s[3]));
        const float alpha = expf(mx - mn);  // 0 for the first group (mx = -inf, mn finite: key kb is always valid)
        float pw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) pw[u] = expf(s[u] - mn);
        l = l * alpha + ((pw[0] + pw[1]) + (pw[2] + pw[3]));
#pragma unroll
        for (int i = 0; i < ND; ++i) {
            float a = acc[i] * alpha;
#pragma unroll
            for (int u = 0; u < 4; ++u) a = fmaf(pw[u], r[u][i], a);
            acc[i] = a;
        }
        mx = mn;
    }
    if (lane == 0) {
        s_m[wave] = mx;
        s_l[wave] = l;
    }
#pragma unroll
    for (int i = 0; i < ND; ++i) s_acc[wave][lane + 64 * i] = acc[i];
    __syncthreads();
    const float M4 = fmaxf(fmaxf(s_m[0], s_m[1]), fmaxf(s_m[2], s_m[3]));
    float wgt[4], L = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        wgt[w] = expf(s_m[w] - M4);  // a wave without keys: exp(-inf) = 0
        L += wgt[w] * s_l[w];
    }
    float* out = ctx + ((size_t)m * H + h) * KR;
    for (int d = threadIdx.x; d < KR; d += blockDim.x) {
        float a = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) a = fmaf(wgt[w], s_acc[w][d], a);
        out[d] = a / L;
    }
}

__global__ __launch_bounds__(256) void row_argmax_kernel(const float* logits, int n, float* max_out, int* idx_out) {
    __shared__ float s_v[4];
    __shared__ int s_i[4];
    const float* row = logits + (size_t)blockIdx.x * n;
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = row[i];
        if (v > best) {  // ascending i per thread: the first maximum stays
            best = v;
            bi = i;
        }
    }
    const float wbest = wave_allmax(best);
    int cand = (best == wbest) ? bi : 0x7fffffff;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) cand = min(cand, __shfl_xor(cand, off, 64));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
        s_v[wave] = wbest;
        s_i[wave] = cand;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float v = s_v[0];
        int ix = s_i[0];
        for (int w = 1; w < 4; ++w)
            if (s_v[w] > v || (s_v[w] == v && s_i[w] < ix)) {
                v = s_v[w];
                ix = s_i[w];
            }
        if (ix == 0x7fffffff) ix = 0;  // a row of NaNs
        if (max_out) max_out[blockIdx.x] = v;
        if (idx_out) idx_out[blockIdx.x] = ix;
    }
}

}  // namespace

int launch_embed(const bf16_t* table, const int* ids, float* x, int M, int W, int vocab, int* flag, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    embed_kernel<<<M, 256, 0, s>>>(table, ids, x, W, vocab, flag);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_norm_shift(const float* x, const float* w, const float* mu, float eps, float* out, int M, int W, const int* row_prev,
                      const int* row_slot, const float* shift_state, size_t slot_stride, const int* row_entry_if_last, float* last_out,
                      hipStream_t s) {
    if (M <= 0) return ZG_OK;
    norm_shift_kernel<<<M, 256, 0, s>>>(x, w, mu, eps, out, W, row_prev, row_slot, shift_state, slot_stride, row_entry_if_last, last_out);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_commit_rows(float* dst, size_t slot_stride, const float* src, size_t src_stride, const int* slots, int n_entries, int width,
                       int n_sets, size_t dst_set_stride, size_t src_set_stride, hipStream_t s) {
    if (n_entries <= 0 || n_sets <= 0) return ZG_OK;
    commit_rows_kernel<<<dim3(n_entries, n_sets), 256, 0, s>>>(dst, slot_stride, src, src_stride, slots, width, dst_set_stride, src_set_stride);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_norm_add(float* x, const float* y, const float* w, float eps, int M, int W, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    norm_add_kernel<<<M, 256, 0, s>>>(x, y, w, eps, W);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_norm_gather(const float* x, const int* rows, const float* w, float eps, float* out, int n_rows, int W, hipStream_t s) {
    if (n_rows <= 0) return ZG_OK;
    norm_gather_kernel<<<n_rows, 256, 0, s>>>(x, rows, w, eps, out, W);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_norm_plain(float* v, int ld, int rows_per_m, int width, int M, const float* w, float eps, hipStream_t s) {
    const int n_vec = M * rows_per_m;
    if (n_vec <= 0) return ZG_OK;
    norm_plain_kernel<<<(n_vec + 3) / 4, 256, 0, s>>>(v, ld, rows_per_m, width, n_vec, w, eps);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_hgrn2_gates(float* proj, int ld, int M, int HD, const float* bias, const float* low, hipStream_t s) {
    const size_t n = (size_t)M * HD;
    if (n == 0) return ZG_OK;
    hgrn2_gates_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(proj, ld, M, HD, bias, low);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_hgrn2_scan(const float* proj, int ld, float* out, int ldo, float* state, size_t slot_stride, const int* ent_start,
                      const int* ent_len, const int* ent_slot, int n_entries, int H, int D, int V, hipStream_t s) {
    if (n_entries <= 0) return ZG_OK;
    ZG_REQUIRE(D >= 1 && D <= 16 * kScanRows, ZG_ERR_UNSUPPORTED, "hgrn2: %d key channels per head (at most %d)", D, 16 * kScanRows);
    int G = 1;
    while (G * kScanRows < D) G <<= 1;
    int threads = ((V * G + 63) / 64) * 64;
    if (threads > 256) threads = 256;
    const int cols = threads / G;
    const dim3 grid(n_entries, H, (V + cols - 1) / cols);
#define ZG_SCAN(G_) hgrn2_scan_kernel<G_><<<grid, threads, 0, s>>>(proj, ld, out, ldo, state, slot_stride, ent_start, ent_len, ent_slot, H, D, V)
    switch (G) {
        case 1: ZG_SCAN(1); break;
        case 2: ZG_SCAN(2); break;
        case 4: ZG_SCAN(4); break;
        case 8: ZG_SCAN(8); break;
        default: ZG_SCAN(16); break;
    }
#undef ZG_SCAN
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_latent_prep(const float* proj, int ld, int M, int q_rank, int KR, int R, const float* wq, const float* wkv, float eps, Rotary rot,
                       const int* row_pos, const int* row_slot, const int* page_table, int max_pages, int page_tokens, float* cq,
                       float* cache, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    ZG_REQUIRE(rot.dims % 2 == 0 && rot.dims <= R, ZG_ERR_ARG, "rotary: %d rotated dimensions of a part of %d", rot.dims, R);
    latent_prep_kernel<<<M, 256, 0, s>>>(proj, ld, q_rank, KR, R, wq, wkv, eps, rot, row_pos, row_slot, page_table, max_pages, page_tokens, cq,
                                         cache);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_q_rotary(const float* q, int ldq, float* qa, int ldqa, int M, int H, int D, int R, int KR, Rotary rot, const int* row_pos,
                    hipStream_t s) {
    if (M <= 0 || R <= 0) return ZG_OK;
    q_rotary_kernel<<<M, 256, 0, s>>>(q, ldq, qa, ldqa, H, D, R, KR, rot, row_pos);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_latent_attention(const float* qa, float* ctx, int M, int H, int KR, int R, float scale, const int* row_pos, const int* row_slot,
                            const int* page_table, int max_pages, int page_tokens, const float* cache, float* ws, size_t ws_floats,
                            hipStream_t s) {
    if (M <= 0) return ZG_OK;
    const int nd = (KR + R + 63) / 64;
    ZG_REQUIRE(nd <= 16, ZG_ERR_UNSUPPORTED, "latent attention: %d cached dimensions per token (at most 1024)", KR + R);
    const dim3 grid(M, H);
#define ZG_ATT(ND_) \
    latent_attention_kernel<ND_><<<grid, 256, 0, s>>>(qa, ctx, H, KR, R, scale, row_pos, row_slot, page_table, max_pages, page_tokens, cache)
    if (nd <= 1) ZG_ATT(1);
    else if (nd <= 2) ZG_ATT(2);
    else if (nd <= 3) ZG_ATT(3);
    else if (nd <= 4) ZG_ATT(4);
    else if (nd <= 6) ZG_ATT(6);
    else if (nd <= 9) ZG_ATT(9);
    else if (nd <= 12) ZG_ATT(12);
    else ZG_ATT(16);
#undef ZG_ATT
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_row_argmax(const float* logits, int rows, int n, float* max_out, int* idx_out, hipStream_t s) {
    if (rows <= 0) return ZG_OK;
    row_argmax_kernel<<<rows, 256, 0, s>>>(logits, n, max_out, idx_out);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

}  // namespace lm
}  // namespace zg
