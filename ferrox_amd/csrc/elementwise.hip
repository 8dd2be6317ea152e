// Row-wise kernels: embedding gather, RMSNorm, rotary + cache write, residual
// add, casts, the weighted sum of routed expert outputs.
//
// The residual stream `h` is float32 in both precisions; normed activations and
// q/k/v are in the activation type T (float or bf16).  Statistics, angles and
// sums are computed in float32.
#include "common.h"

FX_DEFINE_LAST_ERROR()

// ---------------------------------------------------------------------------
// embedding: h[t, :] = table[ids[t], :] * scale   (the reference has no scale, ferrox-models/src/decoder.rs:1279-1284;
// a design that multiplies its embeddings by a constant does so here, in float32)
// ---------------------------------------------------------------------------
template <typename W>
__global__ void embed_kernel(const W* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ h, int H, int V, float scale,
                             const W* __restrict__ pos_table, const int* __restrict__ positions, int n_pos) {
    const int t = blockIdx.x;
    int id = ids[t];
    const int pos = pos_table ? positions[t] : 0;
    if (id < 0 || id >= V || pos < 0 || (pos_table && pos >= n_pos)) {  // the host rejects such ids and places; never read outside a table
        for (int c = threadIdx.x; c < H; c += blockDim.x) h[(size_t)t * H + c] = __int_as_float(0x7fc00000);
        return;
    }
    const W* row = table + (size_t)id * H;
    if (pos_table) {       // a learned vector per position joins the token's row (it is not scaled)
        const W* prow = pos_table + (size_t)pos * H;
        for (int c = threadIdx.x; c < H; c += blockDim.x) h[(size_t)t * H + c] = to_float(row[c]) * scale + to_float(prow[c]);
        return;
    }
    for (int c = threadIdx.x; c < H; c += blockDim.x) h[(size_t)t * H + c] = to_float(row[c]) * scale;
}

FX_API int fx_embed(void* stream, int w_dtype, const void* table, const int* ids, float* h,
                    int T, int H, int V, float scale, const void* pos_table, const int* positions, int n_pos) {
    FX_REQUIRE(T >= 0 && H > 0 && V > 0, "embed: bad sizes T=%d H=%d V=%d", T, H, V);
    FX_REQUIRE(!pos_table || (positions && n_pos > 0), "embed: a table of positions needs the tokens' positions");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (w_dtype == FX_F32)
        embed_kernel<float><<<T, 256, 0, s>>>((const float*)table, ids, h, H, V, scale, (const float*)pos_table, positions, n_pos);
    else if (w_dtype == FX_BF16)
        embed_kernel<bf16><<<T, 256, 0, s>>>((const bf16*)table, ids, h, H, V, scale, (const bf16*)pos_table, positions, n_pos);
    else
        return fx_fail("embed: unknown table dtype %d", w_dtype);
    FX_CHECK_LAUNCH("embed");
    return 0;
}

// ---------------------------------------------------------------------------
// Layer norm with weight and bias: y = (x - mean) / sqrt(var + eps) * w + b, var the mean of the squared
// deviations from the mean (two passes over the row, which the second finds in cache), all in float32.  Input rows are
// float32 (the residual stream), optionally gathered through `rows`; output is T.  One block per row.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void layernorm_kernel(const float* __restrict__ h, const int* __restrict__ rows,
                                                        const void* __restrict__ w, const void* __restrict__ b, int w_dtype,
                                                        T* __restrict__ out, int H, float eps, long ld) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const float* x = h + (size_t)(rows ? rows[r] : r) * ld;
    if (H <= 256 * 16) {   // the row stays in registers: one pass over memory, weight and bias fetched meanwhile
        float xv[16], wv[16], bv[16];
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = threadIdx.x + i * 256;
            xv[i] = c < H ? x[c] : 0.f;
            sum += xv[i];
        }
        load_strided_as_float<16, 256>(w, w_dtype, threadIdx.x, H, wv);
        if (b) load_strided_as_float<16, 256>(b, w_dtype, threadIdx.x, H, bv);
        const float mean = block_sum<4>(sum, red) / (float)H;
        __syncthreads();                               // (`red` is used again)
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float d = threadIdx.x + i * 256 < H ? xv[i] - mean : 0.f;
            ss = fmaf(d, d, ss);
        }
        const float rstd = 1.0f / sqrtf(block_sum<4>(ss, red) / (float)H + eps);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = threadIdx.x + i * 256;
            if (c < H) from_float(out + (size_t)r * H + c, (xv[i] - mean) * rstd * wv[i] + (b ? bv[i] : 0.f));
        }
        return;
    }
    float sum = 0.f;
    for (int c = threadIdx.x; c < H; c += 256) sum += x[c];
    const float mean = block_sum<4>(sum, red) / (float)H;
    __syncthreads();                                   // (`red` is used again)
    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += 256) {
        const float d = x[c] - mean;
        ss = fmaf(d, d, ss);
    }
    const float rstd = 1.0f / sqrtf(block_sum<4>(ss, red) / (float)H + eps);
    for (int c = threadIdx.x; c < H; c += 256)
        from_float(out + (size_t)r * H + c, (x[c] - mean) * rstd * load_as_float(w, w_dtype, c) + (b ? load_as_float(b, w_dtype, c) : 0.f));
}

FX_API int fx_layernorm(void* stream, int out_dtype, const float* h, const int* rows, const void* w, const void* b,
                        int w_dtype, void* out, int R, int H, float eps, long ld) {
    FX_REQUIRE(R >= 0 && H > 0 && w, "layernorm: bad sizes R=%d H=%d", R, H);
    if (ld == 0) ld = H;
    FX_REQUIRE(ld >= H, "layernorm: rows %ld apart hold fewer than %d columns", ld, H);
    FX_REQUIRE(w_dtype == FX_F32 || w_dtype == FX_BF16, "layernorm: unknown weight dtype %d", w_dtype);
    if (R == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == FX_F32) layernorm_kernel<float><<<R, 256, 0, s>>>(h, rows, w, b, w_dtype, (float*)out, H, eps, ld);
    else if (out_dtype == FX_BF16) layernorm_kernel<bf16><<<R, 256, 0, s>>>(h, rows, w, b, w_dtype, (bf16*)out, H, eps, ld);
    else return fx_fail("layernorm: unknown output dtype %d", out_dtype);
    FX_CHECK_LAUNCH("layernorm");
    return 0;
}

// ---------------------------------------------------------------------------
// h += y * sigmoid(g): a sublayer's float32 output rows pass a learned gate, element by element, as they join the
// residual stream.  g holds the gate's logits (float32, a product with its bias added).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gated_add_kernel(float* __restrict__ h, const float* __restrict__ y,
                                                        const float* __restrict__ g, long n) {
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i + 3 < n) {
        const float4 yv = *(const float4*)(y + i), gv = *(const float4*)(g + i);
        float4 hv = *(const float4*)(h + i);
        hv.x += yv.x / (1.0f + expf(-gv.x));
        hv.y += yv.y / (1.0f + expf(-gv.y));
        hv.z += yv.z / (1.0f + expf(-gv.z));
        hv.w += yv.w / (1.0f + expf(-gv.w));
        *(float4*)(h + i) = hv;
        return;
    }
    for (long e = i; e < n; ++e) h[e] += y[e] / (1.0f + expf(-g[e]));
}

FX_API int fx_gated_add(void* stream, float* h, const float* y, const float* g, long n) {
    FX_REQUIRE(n >= 0, "gated_add: %ld elements", n);
    FX_REQUIRE((((uintptr_t)h | (uintptr_t)y | (uintptr_t)g) % 16) == 0, "gated_add: rows must start at multiples of 16 bytes");
    if (n == 0) return 0;
    const long blocks = (n + 1023) / 1024;
    FX_REQUIRE(blocks < (1L << 31), "gated_add: too many elements for one launch");
    gated_add_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(h, y, g, n);
    FX_CHECK_LAUNCH("gated_add");
    return 0;
}

// ---------------------------------------------------------------------------
// RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w, multiply order x*s*w
// (ferrox-core/src/matmul.rs:62-69).  Input rows are float32 (the residual
// stream), optionally gathered through `rows`; output is T.  Without a weight (w null) rows are only
// brought to unit root mean square.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ h, const int* __restrict__ rows,
                                                      const void* __restrict__ w, int w_dtype,
                                                      T* __restrict__ out, int H, float eps, long ld) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const float* x = h + (size_t)(rows ? rows[r] : r) * ld;
    if (H <= 256 * 16) {   // the row stays in registers: one pass over memory, the weights fetched meanwhile
        float xv[16], wv[16];
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = threadIdx.x + i * 256;
            xv[i] = c < H ? x[c] : 0.f;
        }
        if (w) load_strided_as_float<16, 256>(w, w_dtype, threadIdx.x, H, wv);
        else {
#pragma unroll
            for (int i = 0; i < 16; ++i) wv[i] = 1.f;
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) ss += xv[i] * xv[i];
        ss = block_sum<4>(ss, red);
        const float scale = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = threadIdx.x + i * 256;
            if (c < H) from_float(out + (size_t)r * H + c, xv[i] * scale * wv[i]);
        }
        return;
    }
    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += 256) {
        float v = x[c];
        ss += v * v;
    }
    ss = block_sum<4>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)H + eps);
    for (int c = threadIdx.x; c < H; c += 256)
        from_float(out + (size_t)r * H + c, x[c] * scale * (w ? load_as_float(w, w_dtype, c) : 1.f));
}

// Short rows (the heads of q and k, normed one by one): a wave per row, four rows to a block, the row in registers.
// The same sums in another order than the block-wide kernel's, so a row is always normed by the same kernel.
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_short_kernel(const float* __restrict__ h, const int* __restrict__ rows,
                                                            const void* __restrict__ w, int w_dtype,
                                                            T* __restrict__ out, int R, int H, float eps, long ld) {
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (r >= R) return;
    const float* x = h + (size_t)(rows ? rows[r] : r) * ld;
    float xv[4], wv[4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = lane + i * 64;
        xv[i] = c < H ? x[c] : 0.f;
    }
    if (w) load_strided_as_float<4, 64>(w, w_dtype, lane, H, wv);
    else {
#pragma unroll
        for (int i = 0; i < 4; ++i) wv[i] = 1.f;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) ss += xv[i] * xv[i];
    ss = wave_sum(ss);
    const float scale = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = lane + i * 64;
        if (c < H) from_float(out + (size_t)r * H + c, xv[i] * scale * wv[i]);
    }
}

// `ld`: distance between two input rows in floats (0: H, rows that follow each other); the output rows are dense.
FX_API int fx_rmsnorm(void* stream, int out_dtype, const float* h, const int* rows, const void* w,
                      int w_dtype, void* out, int R, int H, float eps, long ld) {
    FX_REQUIRE(R >= 0 && H > 0, "rmsnorm: bad sizes R=%d H=%d", R, H);
    if (ld == 0) ld = H;
    FX_REQUIRE(ld >= H, "rmsnorm: rows %ld apart hold fewer than %d columns", ld, H);
    FX_REQUIRE(w_dtype == FX_F32 || w_dtype == FX_BF16, "rmsnorm: unknown weight dtype %d", w_dtype);
    if (R == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (H <= 256 && (out_dtype == FX_F32 || out_dtype == FX_BF16)) {
        if (out_dtype == FX_F32) rmsnorm_short_kernel<float><<<(R + 3) / 4, 256, 0, s>>>(h, rows, w, w_dtype, (float*)out, R, H, eps, ld);
        else rmsnorm_short_kernel<bf16><<<(R + 3) / 4, 256, 0, s>>>(h, rows, w, w_dtype, (bf16*)out, R, H, eps, ld);
        FX_CHECK_LAUNCH("rmsnorm");
        return 0;
    }
    if (out_dtype == FX_F32)
        rmsnorm_kernel<float><<<R, 256, 0, s>>>(h, rows, w, w_dtype, (float*)out, H, eps, ld);
    else if (out_dtype == FX_BF16)
        rmsnorm_kernel<bf16><<<R, 256, 0, s>>>(h, rows, w, w_dtype, (bf16*)out, H, eps, ld);
    else
        return fx_fail("rmsnorm: unknown output dtype %d", out_dtype);
    FX_CHECK_LAUNCH("rmsnorm");
    return 0;
}

// ---------------------------------------------------------------------------
// Rotary position encoding of q and k, and the write of k and v into the pages.
//
// Split-half pairing (i, i + rot/2), angle = (float)pos * inv_freq[i] in float32, as the reference
// multiplies them (ferrox-core/src/attention.rs:20-32); the caller brings inv_freq[i] = theta^(-2i/rot)
// as a table of rot/2 floats, so that the frequencies are the same numbers wherever they are made.
// `interleaved` pairs (2i, 2i+1) instead.
// `freq_factors` (rot/2 floats, or null): the angle of pair i is divided by freq_factors[i]
// (per-band frequency correction, attention.rs:319-333).
// rot = 0 rotates nothing.  v is never rotated.  Key pages hold
// [page][kv_head][slot][head_dim]; value pages hold the transpose
// [page][kv_head][value head size][slot], which is what the attention kernels read (a value head's size vd
// may differ from head_dim, the size of a query and key head).
// ---------------------------------------------------------------------------
// Values into their transposed pages: block b of ceil(T / 8) * nkv takes eight consecutive tokens of one kv head, so
// that eight tokens that follow each other in one page go out as one 16-byte store per head dimension.
template <typename T>
__device__ __forceinline__ void write_values(int b, const T* __restrict__ v, int ldv, const int* __restrict__ positions,
                                             const int* __restrict__ token_seq, const int* __restrict__ block_table,
                                             int max_blocks, T* __restrict__ v_pages, int n_tokens, int nkv, int bs, int vd) {
    const int tid = threadIdx.x;
    const int kh = b % nkv, t0 = (b / nkv) * 8;
    const int n = min(8, n_tokens - t0);
    const int pos0 = positions[t0], seq0 = token_seq[t0];
    bool together = sizeof(T) == 2 && n == 8 && (bs & 7) == 0 && (pos0 & 7) == 0;
    for (int i = 1; together && i < 8; ++i) together = positions[t0 + i] == pos0 + i && token_seq[t0 + i] == seq0;
    if (together) {
        const int page = block_table[(size_t)seq0 * max_blocks + pos0 / bs];
        T* dst = v_pages + ((size_t)page * nkv + kh) * vd * bs + pos0 % bs;
        for (int d = tid; d < vd; d += 256) {
            uint16_t e[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) e[i] = *(const uint16_t*)(v + (size_t)(t0 + i) * ldv + (size_t)kh * vd + d);
            uint4 o;
            o.x = e[0] | ((uint32_t)e[1] << 16);
            o.y = e[2] | ((uint32_t)e[3] << 16);
            o.z = e[4] | ((uint32_t)e[5] << 16);
            o.w = e[6] | ((uint32_t)e[7] << 16);
            *(uint4*)(dst + (size_t)d * bs) = o;
        }
        return;
    }
    for (int idx = tid; idx < n * vd; idx += 256) {      // tokens of different pages: element by element
        const int i = idx / vd, d = idx - i * vd;
        const int t = t0 + i, pos = positions[t];
        const int page = block_table[(size_t)token_seq[t] * max_blocks + pos / bs];
        v_pages[(((size_t)page * nkv + kh) * vd + d) * bs + pos % bs] = v[(size_t)t * ldv + (size_t)kh * vd + d];
    }
}

// The first T * split blocks rotate: `split` blocks share a token, each computes the angles' sines
// and cosines once and takes its part of the heads of q (in place) and of k (into its page); few
// tokens get several blocks each, many tokens one.  The blocks after them write v: one block per (eight
// consecutive tokens, kv head), so that eight tokens that follow each other in one page go out as
// one 16-byte store per head dimension into the transposed page.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(
    T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
    const int* __restrict__ positions, const int* __restrict__ token_seq,
    const int* __restrict__ block_table, int max_blocks, T* __restrict__ k_pages, T* __restrict__ v_pages,
    int n_tokens, int split, int nh, int nkv, int hd, int bs, int rot, int interleaved, const float* __restrict__ inv_freq, int vec8,
    const float* __restrict__ freq_factors, int vd) {
    __shared__ float cs[128], sn[128];     // rot / 2 <= 128
    const int tid = threadIdx.x;
    const int half = rot >> 1;
    if ((int)blockIdx.x < n_tokens * split) {
        const int t = blockIdx.x / split, part = blockIdx.x % split, step = 256 * split;
        const int pos = positions[t];
        for (int p = tid; p < half; p += 256) {
            float angle = (float)pos * inv_freq[p];
            if (freq_factors) angle = angle / freq_factors[p];
            sincosf(angle, &sn[p], &cs[p]);
        }
        __syncthreads();
        T* k_dst = nullptr;
        if (k_pages) {
            const int page = block_table[(size_t)token_seq[t] * max_blocks + pos / bs];
            k_dst = k_pages + ((size_t)page * nkv * bs + pos % bs) * hd;      // + kv head * bs * hd
        }
        const int heads = nh + (k_pages ? nkv : 0);
        if (vec8) {
            // bfloat16, split halves, everything a multiple of eight: eight neighbouring pairs to a thread, 16 bytes
            // per load and store
            const int h8 = half >> 3;
            for (int i = part * 256 + tid; i < heads * h8; i += step) {
                const int head = i / h8, p = (i - head * h8) * 8;
                const T* src = head < nh ? q + (size_t)t * ldq + (size_t)head * hd : k + (size_t)t * ldk + (size_t)(head - nh) * hd;
                T* dst = head < nh ? q + (size_t)t * ldq + (size_t)head * hd : k_dst + (size_t)(head - nh) * bs * hd;
                const uint4 ua = *(const uint4*)(src + p), ub = *(const uint4*)(src + p + half);
                const uint32_t wa[4] = {ua.x, ua.y, ua.z, ua.w}, wb[4] = {ub.x, ub.y, ub.z, ub.w};
                uint32_t oa[4], ob[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float y0[2], y1[2];
#pragma unroll
                    for (int hh = 0; hh < 2; ++hh) {
                        const float a = __uint_as_float(hh ? wa[e] & 0xffff0000u : wa[e] << 16);
                        const float b = __uint_as_float(hh ? wb[e] & 0xffff0000u : wb[e] << 16);
                        rotate_pair(a, b, cs[p + 2 * e + hh], sn[p + 2 * e + hh], y0[hh], y1[hh]);
                    }
                    oa[e] = pack_bf16(y0[0], y0[1]);
                    ob[e] = pack_bf16(y1[0], y1[1]);
                }
                *(uint4*)(dst + p) = make_uint4(oa[0], oa[1], oa[2], oa[3]);
                *(uint4*)(dst + p + half) = make_uint4(ob[0], ob[1], ob[2], ob[3]);
            }
        } else {
            for (int i = part * 256 + tid; i < heads * half; i += step) {
                const int head = i / half, p = i - head * half;
                const int ia = interleaved ? 2 * p : p;
                const int ib = interleaved ? 2 * p + 1 : p + half;
                const T* src = head < nh ? q + (size_t)t * ldq + (size_t)head * hd : k + (size_t)t * ldk + (size_t)(head - nh) * hd;
                T* dst = head < nh ? q + (size_t)t * ldq + (size_t)head * hd : k_dst + (size_t)(head - nh) * bs * hd;
                const float a = to_float(src[ia]), b = to_float(src[ib]);
                float y0, y1;
                rotate_pair(a, b, cs[p], sn[p], y0, y1);
                from_float(dst + ia, y0);
                from_float(dst + ib, y1);
            }
        }
        if (k_pages && rot < hd) {         // beyond the rotated dimensions
            const int rest = hd - rot;
            for (int i = part * 256 + tid; i < nkv * rest; i += step) {
                const int kh = i / rest, d = rot + i - kh * rest;
                k_dst[(size_t)kh * bs * hd + d] = k[(size_t)t * ldk + (size_t)kh * hd + d];
            }
        }
        return;
    }
    if (!v_pages) return;
    write_values<T>(blockIdx.x - n_tokens * split, v, ldv, positions, token_seq, block_table, max_blocks, v_pages, n_tokens, nkv, bs, vd);
}

FX_API int fx_rope_kv_write(void* stream, int dtype, void* q, int ldq, const void* k, int ldk,
                            const void* v, int ldv, const int* positions, const int* token_seq,
                            const int* block_table, int max_blocks, void* k_pages, void* v_pages,
                            int T, int nh, int nkv, int hd, int bs, int rot, int interleaved, const float* inv_freq,
                            const float* freq_factors, int vd) {
    if (vd <= 0) vd = hd;      // a value head of the keys' size
    FX_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && hd > 0 && bs > 0, "rope_kv_write: bad sizes");
    FX_REQUIRE(rot >= 0 && rot <= hd && rot % 2 == 0, "rope_kv_write: rotary dim %d must be even and <= head_dim %d", rot, hd);
    FX_REQUIRE(rot <= 256, "rope_kv_write: rotary dim %d is more than this kernel's 256", rot);
    FX_REQUIRE(inv_freq || rot == 0, "rope_kv_write: a rotation needs the table of its %d frequencies", rot / 2);
    FX_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "rope_kv_write: key and value pages must come together");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int split = T <= 32 ? 8 : (T <= 128 ? 2 : 1);
    const long n_blocks = (long)T * split + (v_pages ? (long)((T + 7) / 8) * nkv : 0);
    FX_REQUIRE(n_blocks < (1L << 31), "rope_kv_write: too many tokens and heads for one launch");
    const unsigned blocks = (unsigned)n_blocks;
    const int vec8 = dtype == FX_BF16 && !interleaved && rot % 16 == 0 && hd % 8 == 0 && ldq % 8 == 0 && ldk % 8 == 0 &&
                     ((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 && (!k_pages || ((uintptr_t)k_pages % 16) == 0);
    if (dtype == FX_F32)
        rope_kv_write_kernel<float><<<blocks, 256, 0, s>>>((float*)q, ldq, (const float*)k, ldk, (const float*)v, ldv,
                                                           positions, token_seq, block_table, max_blocks,
                                                           (float*)k_pages, (float*)v_pages, T, split, nh, nkv, hd, bs, rot,
                                                           interleaved, inv_freq, 0, freq_factors, vd);
    else if (dtype == FX_BF16)
        rope_kv_write_kernel<bf16><<<blocks, 256, 0, s>>>((bf16*)q, ldq, (const bf16*)k, ldk, (const bf16*)v, ldv,
                                                          positions, token_seq, block_table, max_blocks,
                                                          (bf16*)k_pages, (bf16*)v_pages, T, split, nh, nkv, hd, bs, rot,
                                                          interleaved, inv_freq, vec8, freq_factors, vd);
    else
        return fx_fail("rope_kv_write: unknown dtype %d", dtype);
    FX_CHECK_LAUNCH("rope_kv_write");
    return 0;
}

// ---------------------------------------------------------------------------
// Mixers whose q and k heads go through an RMS norm and are not rotated: one launch norms every head of the
// float32 q/k product, writes q in the activation type, k into its page and v into its transposed page.
//   qk [T, (nh + nkv) * hd] float32: per token nh heads of q, then nkv heads of k (nkv_in = 0: no keys, q alone).
//   y = x / sqrt(mean(x^2) + eps) (* w[d] with a weight of hd elements; wq for q's heads, wk for k's).
// A wave per (token, head), four to a block, the head in registers (hd <= 256): the same sums in the same order as
// the norm kernel for short rows.  The blocks after them write v (write_values).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void head_norm_kv_write_kernel(
    const float* __restrict__ qk, long ldqk, T* __restrict__ q_out, long ldq, const T* __restrict__ v, int ldv,
    const void* __restrict__ wq, const void* __restrict__ wk, int w_dtype, float eps,
    const int* __restrict__ positions, const int* __restrict__ token_seq, const int* __restrict__ block_table, int max_blocks,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int n_tokens, int nh, int nkv, int hd, int bs, int vd, int norm_blocks) {
    if ((int)blockIdx.x >= norm_blocks) {
        if (v_pages) write_values<T>(blockIdx.x - norm_blocks, v, ldv, positions, token_seq, block_table, max_blocks, v_pages, n_tokens, nkv, bs, vd);
        return;
    }
    const int heads = nh + (k_pages ? nkv : 0);
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (r >= n_tokens * heads) return;
    const int t = r / heads, head = r - t * heads;
    const float* x = qk + (size_t)t * ldqk + (size_t)head * hd;
    const void* w = head < nh ? wq : wk;
    float xv[4], wv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = lane + i * 64;
        xv[i] = c < hd ? x[c] : 0.f;
    }
    if (w) load_strided_as_float<4, 64>(w, w_dtype, lane, hd, wv);
    else {
#pragma unroll
        for (int i = 0; i < 4; ++i) wv[i] = 1.f;
    }
    T* dst;
    if (head < nh) dst = q_out + (size_t)t * ldq + (size_t)head * hd;
    else {
        const int pos = positions[t];
        const int page = block_table[(size_t)token_seq[t] * max_blocks + pos / bs];
        dst = k_pages + (((size_t)page * nkv + (head - nh)) * bs + pos % bs) * hd;
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) ss += xv[i] * xv[i];
    ss = wave_sum(ss);
    const float scale = 1.0f / sqrtf(ss / (float)hd + eps);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = lane + i * 64;
        if (c < hd) from_float(dst + c, xv[i] * scale * wv[i]);
    }
}

FX_API int fx_head_norm_kv_write(void* stream, int dtype, const float* qk, long ldqk, void* q_out, long ldq, const void* v, int ldv,
                                 const void* wq, const void* wk, int w_dtype, float eps, const int* positions,
                                 const int* token_seq, const int* block_table, int max_blocks, void* k_pages, void* v_pages,
                                 int T, int nh, int nkv, int hd, int bs, int vd) {
    if (vd <= 0) vd = hd;
    FX_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && bs > 0, "head_norm_kv_write: bad sizes");
    FX_REQUIRE(hd > 0 && hd <= 256, "head_norm_kv_write: head size %d is outside 1..256", hd);
    FX_REQUIRE(w_dtype == FX_F32 || w_dtype == FX_BF16, "head_norm_kv_write: unknown weight dtype %d", w_dtype);
    FX_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "head_norm_kv_write: key and value pages must come together");
    FX_REQUIRE(!v_pages || v, "head_norm_kv_write: value pages without values");
    if (T == 0) return 0;
    const long heads = nh + (k_pages ? nkv : 0);
    const long norm_blocks = (T * heads + 3) / 4, n_blocks = norm_blocks + (v_pages ? (long)((T + 7) / 8) * nkv : 0);
    FX_REQUIRE(n_blocks < (1L << 31), "head_norm_kv_write: too many tokens and heads for one launch");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FX_F32)
        head_norm_kv_write_kernel<float><<<(unsigned)n_blocks, 256, 0, s>>>(qk, ldqk, (float*)q_out, ldq, (const float*)v, ldv, wq, wk,
            w_dtype, eps, positions, token_seq, block_table, max_blocks, (float*)k_pages, (float*)v_pages, T, nh, nkv, hd, bs, vd, (int)norm_blocks);
    else if (dtype == FX_BF16)
        head_norm_kv_write_kernel<bf16><<<(unsigned)n_blocks, 256, 0, s>>>(qk, ldqk, (bf16*)q_out, ldq, (const bf16*)v, ldv, wq, wk,
            w_dtype, eps, positions, token_seq, block_table, max_blocks, (bf16*)k_pages, (bf16*)v_pages, T, nh, nkv, hd, bs, vd, (int)norm_blocks);
    else
        return fx_fail("head_norm_kv_write: unknown dtype %d", dtype);
    FX_CHECK_LAUNCH("head_norm_kv_write");
    return 0;
}

// ---------------------------------------------------------------------------
// For attention that rotates nothing, warms its queries with the position and keeps values of unit size.  From the
// float32 product qkv [T, nh hd | nkv hd | nkv vd | n_gate] of a token at position p:
//   q_out[:, :nh hd]  = q * (1 + coef ln(floor((p + 1) / every) + 1))          the query's temperature (coef 0: none)
//   q_out[:, nh hd:]  = the n_gate gate columns, as they are (the attention kernels read them beside the queries)
//   key page          <- k
//   value page        <- v / sqrt(mean(v^2) + eps) per head (unit_values), else v; transposed
// q_out and the pages have type T; temperature and norm are float32 arithmetic.  The first blocks take (token, unit)
// pairs a wave each, a unit being a head of q, a head of k or the gate columns; the blocks after them take (eight
// consecutive tokens, kv head): they norm the eight value heads into LDS and write them as `write_values` does.
// ---------------------------------------------------------------------------
#define UNIT_VD_MAX 256
template <typename T>
__global__ __launch_bounds__(256) void temp_unit_kv_write_kernel(
    const float* __restrict__ qkv, long ld, T* __restrict__ q_out, long ldq, const int* __restrict__ positions,
    const int* __restrict__ token_seq, const int* __restrict__ block_table, int max_blocks, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int n_tokens, int nh, int nkv, int hd, int vd, int bs, int n_gate, float coef, int every,
    int unit_values, float eps, int head_blocks) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if ((int)blockIdx.x < head_blocks) {
        const int units = nh + (k_pages ? nkv : 0) + (n_gate ? 1 : 0);
        const int r = blockIdx.x * 4 + wave;
        if (r >= n_tokens * units) return;
        const int t = r / units, u = r - t * units;
        const float* row = qkv + (size_t)t * ld;
        if (u < nh) {
            const int pos = positions[t];
            const float temp = coef != 0.f ? 1.0f + coef * logf((float)((pos + 1) / every) + 1.0f) : 1.0f;
            for (int c = lane; c < hd; c += 64) from_float(q_out + (size_t)t * ldq + (size_t)u * hd + c, row[(size_t)u * hd + c] * temp);
        } else if (k_pages && u < nh + nkv) {
            const int kh = u - nh, pos = positions[t];
            const int page = block_table[(size_t)token_seq[t] * max_blocks + pos / bs];
            T* dst = k_pages + (((size_t)page * nkv + kh) * bs + pos % bs) * hd;
            for (int c = lane; c < hd; c += 64) from_float(dst + c, row[(size_t)(nh + kh) * hd + c]);
        } else {
            const float* g = row + (size_t)(nh + nkv) * hd + (size_t)nkv * vd;
            for (int c = lane; c < n_gate; c += 64) from_float(q_out + (size_t)t * ldq + (size_t)nh * hd + c, g[c]);
        }
        return;
    }
    if (!v_pages) return;
    __shared__ T vs[8][UNIT_VD_MAX];
    const int b = blockIdx.x - head_blocks;
    const int kh = b % nkv, t0 = (b / nkv) * 8;
    const int n = min(8, n_tokens - t0);
    for (int i = wave; i < n; i += 4) {
        const float* v = qkv + (size_t)(t0 + i) * ld + (size_t)(nh + nkv) * hd + (size_t)kh * vd;
        float xv[UNIT_VD_MAX / 64];
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < UNIT_VD_MAX / 64; ++e) {
            const int c = lane + e * 64;
            xv[e] = c < vd ? v[c] : 0.f;
            ss = fmaf(xv[e], xv[e], ss);
        }
        const float scale = unit_values ? 1.0f / sqrtf(wave_sum(ss) / (float)vd + eps) : 1.0f;
#pragma unroll
        for (int e = 0; e < UNIT_VD_MAX / 64; ++e) {
            const int c = lane + e * 64;
            if (c < vd) from_float(&vs[i][c], xv[e] * scale);
        }
    }
    __syncthreads();
    const int pos0 = positions[t0], seq0 = token_seq[t0];
    bool together = sizeof(T) == 2 && n == 8 && (bs & 7) == 0 && (pos0 & 7) == 0;
    for (int i = 1; together && i < 8; ++i) together = positions[t0 + i] == pos0 + i && token_seq[t0 + i] == seq0;
    if (together) {      // eight tokens that follow each other in one page: one 16-byte store per value channel
        const int page = block_table[(size_t)seq0 * max_blocks + pos0 / bs];
        T* dst = v_pages + ((size_t)page * nkv + kh) * vd * bs + pos0 % bs;
        for (int d = tid; d < vd; d += 256) {
            uint16_t e[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) e[i] = *(const uint16_t*)&vs[i][d];
            uint4 o;
            o.x = e[0] | ((uint32_t)e[1] << 16);
            o.y = e[2] | ((uint32_t)e[3] << 16);
            o.z = e[4] | ((uint32_t)e[5] << 16);
            o.w = e[6] | ((uint32_t)e[7] << 16);
            *(uint4*)(dst + (size_t)d * bs) = o;
        }
        return;
    }
    for (int idx = tid; idx < n * vd; idx += 256) {
        const int i = idx / vd, d = idx - i * vd;
        const int t = t0 + i, pos = positions[t];
        const int page = block_table[(size_t)token_seq[t] * max_blocks + pos / bs];
        v_pages[(((size_t)page * nkv + kh) * vd + d) * bs + pos % bs] = vs[i][d];
    }
}

FX_API int fx_temp_unit_kv_write(void* stream, int dtype, const float* qkv, long ld, void* q_out, long ldq, const int* positions,
                                 const int* token_seq, const int* block_table, int max_blocks, void* k_pages, void* v_pages,
                                 int T, int nh, int nkv, int hd, int vd, int bs, int n_gate, float coef, int every,
                                 int unit_values, float eps) {
    FX_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && bs > 0 && n_gate >= 0, "temp_unit_kv_write: bad sizes");
    FX_REQUIRE(hd > 0 && vd > 0 && vd <= UNIT_VD_MAX, "temp_unit_kv_write: head sizes %d and %d (values up to %d)", hd, vd, UNIT_VD_MAX);
    FX_REQUIRE(every >= 1, "temp_unit_kv_write: a temperature step every %d positions", every);
    FX_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "temp_unit_kv_write: key and value pages must come together");
    FX_REQUIRE(ld >= (long)(nh + nkv) * hd + (long)nkv * vd + n_gate && ldq >= (long)nh * hd + n_gate, "temp_unit_kv_write: rows too short");
    if (T == 0) return 0;
    const long units = nh + (k_pages ? nkv : 0) + (n_gate ? 1 : 0);
    const long head_blocks = (T * units + 3) / 4, n_blocks = head_blocks + (v_pages ? (long)((T + 7) / 8) * nkv : 0);
    FX_REQUIRE(n_blocks < (1L << 31), "temp_unit_kv_write: too many tokens and heads for one launch");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FX_F32)
        temp_unit_kv_write_kernel<float><<<(unsigned)n_blocks, 256, 0, s>>>(qkv, ld, (float*)q_out, ldq, positions, token_seq, block_table,
            max_blocks, (float*)k_pages, (float*)v_pages, T, nh, nkv, hd, vd, bs, n_gate, coef, every, unit_values, eps, (int)head_blocks);
    else if (dtype == FX_BF16)
        temp_unit_kv_write_kernel<bf16><<<(unsigned)n_blocks, 256, 0, s>>>(qkv, ld, (bf16*)q_out, ldq, positions, token_seq, block_table,
            max_blocks, (bf16*)k_pages, (bf16*)v_pages, T, nh, nkv, hd, vd, bs, n_gate, coef, every, unit_values, eps, (int)head_blocks);
    else
        return fx_fail("temp_unit_kv_write: unknown dtype %d", dtype);
    FX_CHECK_LAUNCH("temp_unit_kv_write");
    return 0;
}

// ---------------------------------------------------------------------------
// The gated add and the layer norm that follows it, one launch: h += y * sigmoid(g), then
// out = (h - mean) / sqrt(var + eps) * w + b of the new row.  Rows of up to 4,096 columns stay in registers; the
// sums are those of the two kernels it stands for (the same order, so the same bits).  One block per row.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gated_add_layernorm_kernel(float* __restrict__ h, const float* __restrict__ y,
                                                                  const float* __restrict__ g, const void* __restrict__ w,
                                                                  const void* __restrict__ b, int w_dtype, T* __restrict__ out,
                                                                  int H, float eps) {
    __shared__ float red[4];
    const size_t row = (size_t)blockIdx.x * H;
    float xv[16], wv[16], bv[16];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int c = threadIdx.x + i * 256;
        xv[i] = 0.f;
        if (c < H) {
            xv[i] = h[row + c] + y[row + c] / (1.0f + expf(-g[row + c]));
            h[row + c] = xv[i];
        }
        sum += xv[i];
    }
    load_strided_as_float<16, 256>(w, w_dtype, threadIdx.x, H, wv);
    if (b) load_strided_as_float<16, 256>(b, w_dtype, threadIdx.x, H, bv);
    const float mean = block_sum<4>(sum, red) / (float)H;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float d = threadIdx.x + i * 256 < H ? xv[i] - mean : 0.f;
        ss = fmaf(d, d, ss);
    }
    const float rstd = 1.0f / sqrtf(block_sum<4>(ss, red) / (float)H + eps);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int c = threadIdx.x + i * 256;
        if (c < H) from_float(out + row + c, (xv[i] - mean) * rstd * wv[i] + (b ? bv[i] : 0.f));
    }
}

FX_API int fx_gated_add_layernorm(void* stream, int out_dtype, float* h, const float* y, const float* g, const void* w,
                                  const void* b, int w_dtype, void* out, int T, int H, float eps) {
    FX_REQUIRE(T >= 0 && H > 0 && H <= 4096 && w, "gated_add_layernorm: %d rows of %d columns (up to 4096)", T, H);
    FX_REQUIRE(w_dtype == FX_F32 || w_dtype == FX_BF16, "gated_add_layernorm: unknown weight dtype %d", w_dtype);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == FX_F32) gated_add_layernorm_kernel<float><<<T, 256, 0, s>>>(h, y, g, w, b, w_dtype, (float*)out, H, eps);
    else if (out_dtype == FX_BF16) gated_add_layernorm_kernel<bf16><<<T, 256, 0, s>>>(h, y, g, w, b, w_dtype, (bf16*)out, H, eps);
    else return fx_fail("gated_add_layernorm: unknown output dtype %d", out_dtype);
    FX_CHECK_LAUNCH("gated_add_layernorm");
    return 0;
}

// ---------------------------------------------------------------------------
// Latent attention, what a layer keeps per position.  `down` [T, R + rd] float32 is the down-projection of a
// token: R latent channels, then a key part of rd dimensions that all heads share.  One block per token:
//   c = down[:R] / sqrt(mean(down[:R]^2) + eps) * w          (statistics and product in float32)
//   kr = the key part with the pairs (2i, 2i+1), i < rot / 2, turned by pos * inv_freq[i] and stretched by
//        `magnitude` (cosine and sine are both multiplied by it); dimensions from rot on pass
// The key page [page][1][slot][R + rd] receives (c | kr): a query row (its part that went through the keys'
// up-projection | its rotated part) then scores against it as against the key of one shared head.  The value
// page [page][1][R][slot] receives c transposed: the heads' outputs are sums of latents, which the values'
// up-projection is applied to afterwards.
// With `q_src` (the queries' down-projection of the same tokens, [T, Rq] float32, usually the columns beside `down` in
// one product's output) a second row of blocks norms that latent too, q_out[t] = q_src[t] / rms * q_w in the pages'
// type: the two norms that follow the down-projection are one launch.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(
    const float* __restrict__ down, long ldd, const void* __restrict__ w, int w_dtype, float eps,
    const int* __restrict__ positions, const int* __restrict__ token_seq, const int* __restrict__ block_table, int max_blocks,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int R, int rd, int rot, int bs, const float* __restrict__ inv_freq,
    float magnitude, const float* __restrict__ q_src, long ldqs, const void* __restrict__ q_w, float q_eps,
    T* __restrict__ q_out, long ldq, int Rq) {
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    if (blockIdx.y == 1) {          // the queries' latent
        const float* xq = q_src + (size_t)t * ldqs;
        float sq = 0.f;
        for (int c = tid; c < Rq; c += 256) sq = fmaf(xq[c], xq[c], sq);
        sq = block_sum<4>(sq, red);
        const float qs = 1.0f / sqrtf(sq / (float)Rq + q_eps);
        for (int c = tid; c < Rq; c += 256) from_float(q_out + (size_t)t * ldq + c, xq[c] * qs * load_as_float(q_w, w_dtype, c));
        return;
    }
    const float* x = down + (size_t)t * ldd;
    const int pos = positions[t];
    const int page = block_table[(size_t)token_seq[t] * max_blocks + pos / bs], slot = pos % bs;
    T* k_dst = k_pages + ((size_t)page * bs + slot) * (R + rd);
    T* v_dst = v_pages + (size_t)page * R * bs + slot;        // + channel * bs
    float ss = 0.f;
    for (int c = tid; c < R; c += 256) ss = fmaf(x[c], x[c], ss);
    ss = block_sum<4>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)R + eps);
    for (int c = tid; c < R; c += 256) {
        T y;
        from_float(&y, x[c] * scale * load_as_float(w, w_dtype, c));
        k_dst[c] = y;
        v_dst[(size_t)c * bs] = y;
    }
    const int half = rot >> 1;
    for (int p = tid; p < half; p += 256) {
        float sn, cs, y0, y1;
        sincosf((float)pos * inv_freq[p], &sn, &cs);
        rotate_pair(x[R + 2 * p], x[R + 2 * p + 1], cs * magnitude, sn * magnitude, y0, y1);
        from_float(k_dst + R + 2 * p, y0);
        from_float(k_dst + R + 2 * p + 1, y1);
    }
    for (int d = rot + tid; d < rd; d += 256) from_float(k_dst + R + d, x[R + d]);
}

FX_API int fx_latent_kv_write(void* stream, int dtype, const float* down, long ldd, const void* w, int w_dtype, float eps,
                              const int* positions, const int* token_seq, const int* block_table, int max_blocks,
                              void* k_pages, void* v_pages, int T, int R, int rd, int rot, int bs, const float* inv_freq,
                              float magnitude, const float* q_src, long ldqs, const void* q_w, float q_eps, void* q_out,
                              long ldq, int Rq) {
    FX_REQUIRE(T >= 0 && R > 0 && rd >= 0 && bs > 0 && ldd >= R + rd, "latent_kv_write: bad sizes T=%d R=%d rd=%d", T, R, rd);
    FX_REQUIRE(rot >= 0 && rot <= rd && rot % 2 == 0, "latent_kv_write: %d rotated dimensions of %d", rot, rd);
    FX_REQUIRE(inv_freq || rot == 0, "latent_kv_write: a rotation needs the table of its %d frequencies", rot / 2);
    FX_REQUIRE(w_dtype == FX_F32 || w_dtype == FX_BF16, "latent_kv_write: unknown weight dtype %d", w_dtype);
    FX_REQUIRE(k_pages && v_pages && w, "latent_kv_write: pages and the norm's weight are needed");
    FX_REQUIRE(!q_src || (q_w && q_out && Rq > 0 && ldqs >= Rq && ldq >= Rq), "latent_kv_write: the queries' latent needs a weight, an output and %d columns", Rq);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(T, q_src ? 2 : 1);
    if (dtype == FX_F32)
        latent_kv_write_kernel<float><<<grid, 256, 0, s>>>(down, ldd, w, w_dtype, eps, positions, token_seq, block_table, max_blocks,
                                                           (float*)k_pages, (float*)v_pages, R, rd, rot, bs, inv_freq, magnitude,
                                                           q_src, ldqs, q_w, q_eps, (float*)q_out, ldq, Rq);
    else if (dtype == FX_BF16)
        latent_kv_write_kernel<bf16><<<grid, 256, 0, s>>>(down, ldd, w, w_dtype, eps, positions, token_seq, block_table, max_blocks,
                                                          (bf16*)k_pages, (bf16*)v_pages, R, rd, rot, bs, inv_freq, magnitude,
                                                          q_src, ldqs, q_w, q_eps, (bf16*)q_out, ldq, Rq);
    else
        return fx_fail("latent_kv_write: unknown dtype %d", dtype);
    FX_CHECK_LAUNCH("latent_kv_write");
    return 0;
}

// The rotated part of the queries of latent attention: q [T, nh * (D + rd)] holds per head D dimensions that are
// not rotated and rd that are; the rd are turned as the shared key part is (pairs (2i, 2i+1), i < rot / 2, by
// pos * inv_freq[i], stretched by `magnitude`) and written behind the first R columns of that head's row of
// q_lat [T, nh * (R + rd)] (the first R columns hold the unrotated part taken through the keys' up-projection, from a
// matrix product).  q_lat may be q itself (D = R: rotation in place; a thread reads the elements it writes, and no
// other).  One block per token.
template <typename T>
__global__ __launch_bounds__(256) void latent_q_rot_kernel(const T* q, long ldq, T* q_lat, long ldl,
                                                           const int* __restrict__ positions, int nh, int D, int rd, int rot, int R,
                                                           const float* __restrict__ inv_freq, float magnitude) {
    __shared__ float cs[128], sn[128];
    const int t = blockIdx.x, tid = threadIdx.x, half = rot >> 1;
    const int pos = positions[t];
    for (int p = tid; p < half; p += 256) {
        float s_, c_;
        sincosf((float)pos * inv_freq[p], &s_, &c_);
        cs[p] = c_ * magnitude;
        sn[p] = s_ * magnitude;
    }
    __syncthreads();
    for (int i = tid; i < nh * half; i += 256) {
        const int h = i / half, p = i - h * half;
        const T* src = q + (size_t)t * ldq + (size_t)h * (D + rd) + D;
        T* dst = q_lat + (size_t)t * ldl + (size_t)h * (R + rd) + R;
        float y0, y1;
        rotate_pair(to_float(src[2 * p]), to_float(src[2 * p + 1]), cs[p], sn[p], y0, y1);
        from_float(dst + 2 * p, y0);
        from_float(dst + 2 * p + 1, y1);
    }
    const int rest = rd - rot;
    for (int i = tid; i < nh * rest; i += 256) {
        const int h = i / rest, d = rot + i - h * rest;
        q_lat[(size_t)t * ldl + (size_t)h * (R + rd) + R + d] = q[(size_t)t * ldq + (size_t)h * (D + rd) + D + d];
    }
}

FX_API int fx_latent_q_rot(void* stream, int dtype, const void* q, long ldq, void* q_lat, long ldl, const int* positions,
                           int T, int nh, int D, int rd, int rot, int R, const float* inv_freq, float magnitude) {
    FX_REQUIRE(T >= 0 && nh > 0 && D >= 0 && rd >= 0 && R > 0, "latent_q_rot: bad sizes");
    FX_REQUIRE(ldq >= (long)nh * (D + rd) && ldl >= (long)nh * (R + rd), "latent_q_rot: rows shorter than %d heads", nh);
    FX_REQUIRE(rot >= 0 && rot <= rd && rot % 2 == 0 && rot <= 256, "latent_q_rot: %d rotated dimensions of %d", rot, rd);
    FX_REQUIRE(inv_freq || rot == 0, "latent_q_rot: a rotation needs the table of its %d frequencies", rot / 2);
    if (T == 0 || rd == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FX_F32)
        latent_q_rot_kernel<float><<<T, 256, 0, s>>>((const float*)q, ldq, (float*)q_lat, ldl, positions, nh, D, rd, rot, R, inv_freq, magnitude);
    else if (dtype == FX_BF16)
        latent_q_rot_kernel<bf16><<<T, 256, 0, s>>>((const bf16*)q, ldq, (bf16*)q_lat, ldl, positions, nh, D, rd, rot, R, inv_freq, magnitude);
    else
        return fx_fail("latent_q_rot: unknown dtype %d", dtype);
    FX_CHECK_LAUNCH("latent_q_rot");
    return 0;
}

// ---------------------------------------------------------------------------
// Queries and keys normed over their whole projection, keys that are their own values.  From the float32 product
// qk [T, nh * hd + nkv * hd] (a token's queries, then its keys), one launch writes
//   q_out [T, nh * hd]: the queries normed over all nh * hd columns, x / sqrt(mean + eps) * wq[column]
//   the key page: the keys normed over all nkv * hd columns with wk
//   the transposed value page: the keys as they are, not normed
// Blocks (token, 0) take the queries, blocks (token, 1) the keys (left out when there are no pages to write).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void span_norm_kv_write_kernel(
    const float* __restrict__ qk, long ldqk, T* __restrict__ q_out, long ldq, const void* __restrict__ wq,
    const void* __restrict__ wk, int w_dtype, float eps,
    const int* __restrict__ positions, const int* __restrict__ token_seq, const int* __restrict__ block_table, int max_blocks,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int nh, int nkv, int hd, int bs) {
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    const bool keys = blockIdx.y == 1;
    const int n = (keys ? nkv : nh) * hd;
    const float* x = qk + (size_t)t * ldqk + (keys ? (size_t)nh * hd : 0);
    const void* w = keys ? wk : wq;
    float ss = 0.f;
    for (int c = tid; c < n; c += 256) ss = fmaf(x[c], x[c], ss);
    ss = block_sum<4>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)n + eps);
    if (!keys) {
        for (int c = tid; c < n; c += 256) from_float(q_out + (size_t)t * ldq + c, x[c] * scale * load_as_float(w, w_dtype, c));
        return;
    }
    const int pos = positions[t];
    const int page = block_table[(size_t)token_seq[t] * max_blocks + pos / bs], slot = pos % bs;
    for (int c = tid; c < n; c += 256) {
        const int g = c / hd, d = c - g * hd;
        from_float(k_pages + (((size_t)page * nkv + g) * bs + slot) * hd + d, x[c] * scale * load_as_float(w, w_dtype, c));
        from_float(v_pages + (((size_t)page * nkv + g) * hd + d) * bs + slot, x[c]);
    }
}

FX_API int fx_span_norm_kv_write(void* stream, int dtype, const float* qk, long ldqk, void* q_out, long ldq, const void* wq,
                                 const void* wk, int w_dtype, float eps, const int* positions, const int* token_seq,
                                 const int* block_table, int max_blocks, void* k_pages, void* v_pages, int T, int nh, int nkv,
                                 int hd, int bs) {
    FX_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && hd > 0 && bs > 0, "span_norm_kv_write: bad sizes");
    FX_REQUIRE(ldq >= (long)nh * hd && ldqk >= (long)(nh + (k_pages ? nkv : 0)) * hd, "span_norm_kv_write: rows shorter than their heads");
    FX_REQUIRE(w_dtype == FX_F32 || w_dtype == FX_BF16, "span_norm_kv_write: unknown weight dtype %d", w_dtype);
    FX_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "span_norm_kv_write: key and value pages must come together");
    FX_REQUIRE(wq && (wk || !k_pages), "span_norm_kv_write: the norms' weights are needed");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(T, k_pages ? 2 : 1);
    if (dtype == FX_F32)
        span_norm_kv_write_kernel<float><<<grid, 256, 0, s>>>(qk, ldqk, (float*)q_out, ldq, wq, wk, w_dtype, eps, positions, token_seq,
                                                              block_table, max_blocks, (float*)k_pages, (float*)v_pages, nh, nkv, hd, bs);
    else if (dtype == FX_BF16)
        span_norm_kv_write_kernel<bf16><<<grid, 256, 0, s>>>(qk, ldqk, (bf16*)q_out, ldq, wq, wk, w_dtype, eps, positions, token_seq,
                                                             block_table, max_blocks, (bf16*)k_pages, (bf16*)v_pages, nh, nkv, hd, bs);
    else
        return fx_fail("span_norm_kv_write: unknown dtype %d", dtype);
    FX_CHECK_LAUNCH("span_norm_kv_write");
    return 0;
}

// ---------------------------------------------------------------------------
// h[t, :] += y[t, :]  (float32 sum), y of either type.  Used by parts that have
// no fused epilogue of their own.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ h, const T* __restrict__ y, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) h[i] += to_float(y[i]);
}

FX_API int fx_residual_add(void* stream, int y_dtype, float* h, const void* y, long n) {
    FX_REQUIRE(n >= 0, "residual_add: bad size");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 65536) blocks = 65536;
    if (y_dtype == FX_F32)
        residual_add_kernel<float><<<blocks, 256, 0, s>>>(h, (const float*)y, (size_t)n);
    else if (y_dtype == FX_BF16)
        residual_add_kernel<bf16><<<blocks, 256, 0, s>>>(h, (const bf16*)y, (size_t)n);
    else
        return fx_fail("residual_add: unknown dtype %d", y_dtype);
    FX_CHECK_LAUNCH("residual_add");
    return 0;
}

// ---------------------------------------------------------------------------
// casts between float32 and bf16
// ---------------------------------------------------------------------------
template <typename A, typename B>
__global__ void cast_kernel(const A* __restrict__ a, B* __restrict__ b, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) from_float(b + i, to_float(a[i]));
}

FX_API int fx_cast(void* stream, int src_dtype, const void* src, int dst_dtype, void* dst, long n) {
    FX_REQUIRE(n >= 0, "cast: bad size");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 65536) blocks = 65536;
    if (src_dtype == FX_F32 && dst_dtype == FX_BF16)
        cast_kernel<float, bf16><<<blocks, 256, 0, s>>>((const float*)src, (bf16*)dst, (size_t)n);
    else if (src_dtype == FX_BF16 && dst_dtype == FX_F32)
        cast_kernel<bf16, float><<<blocks, 256, 0, s>>>((const bf16*)src, (float*)dst, (size_t)n);
    else
        return fx_fail("cast: unsupported pair %d -> %d", src_dtype, dst_dtype);
    FX_CHECK_LAUNCH("cast");
    return 0;
}

// ---------------------------------------------------------------------------
// Weighted sum of the routed experts' outputs into the residual stream:
//   h[t, :] += sum_j w[t, j] * y[inv[t*k + j], :]      (inv null: y[t*k + j, :])
//              + gate[t] * shared[t, :]                  (if a shared expert's output is given)
// in ascending j, the selection order (ferrox-moe/src/lib.rs:735-745).
// y is float32 [T*k, H].
// ---------------------------------------------------------------------------
// xg != nullptr: the new rows are also written as xg = round(h * norm_w) (no scale yet) with each block's sum
// of squares of its 256 columns in ss[t * gridDim.y + blockIdx.y]: the product that reads xg scales its
// rows by rsqrt(sum / H + eps), which is RMSNorm with the rounding of the norm that a product applies itself.
// VEC = 4: a thread takes four neighbouring columns with 16-byte loads (H % 4 == 0, aligned rows); a block then
// covers 1024 columns, and each of its waves one group of 256 for the sums of squares.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ h, const float* __restrict__ y,
                                                          const int* __restrict__ inv, const float* __restrict__ w,
                                                          const float* __restrict__ shared, const float* __restrict__ gate,
                                                          int H, int k, int slabs, const void* __restrict__ norm_w,
                                                          int norm_dtype, T* __restrict__ xg, float* __restrict__ ss) {
    __shared__ float red[4];
    const int t = blockIdx.x, n_tok = gridDim.x;
    const int c = (blockIdx.y * 256 + threadIdx.x) * VEC;
    auto load = [&](const float* p, float (&out)[VEC]) {
        if constexpr (VEC == 4) {
            const float4 q = *(const float4*)p;
            out[0] = q.x; out[1] = q.y; out[2] = q.z; out[3] = q.w;
        } else {
            out[0] = *p;
        }
    };
    float v[VEC], nw[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = nw[i] = 0.f;
    if (c < H) {
        // the loads of eight terms are asked for together and added in order: the sums are those of a plain loop
        float h_old[VEC], acc[VEC];
        load(h + (size_t)t * H + c, h_old);
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
        for (int j0 = 0; j0 < k; j0 += 8) {
            float wv[8], yv[8][VEC];
            int from[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int j = min(j0 + u, k - 1);
                from[u] = inv ? inv[t * k + j] : t * k + j;
                wv[u] = w[t * k + j];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) load(y + (size_t)from[u] * H + c, yv[u]);
            if (j0 == 0 && xg) {     // (waits for its load: after the others have left)
#pragma unroll
                for (int i = 0; i < VEC; ++i) nw[i] = load_as_float(norm_w, norm_dtype, c + i);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (j0 + u < k) {
#pragma unroll
                    for (int i = 0; i < VEC; ++i) acc[i] = fmaf(wv[u], yv[u][i], acc[i]);
                }
        }
        if (shared) {      // routed first, then shared (lib.rs:746-750); the shared output may come as `slabs` partial sums [slab][T][H]
            float sh[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) sh[i] = 0.f;
            for (int s0 = 0; s0 < slabs; s0 += 8) {
                float sv[8][VEC];
#pragma unroll
                for (int u = 0; u < 8; ++u) load(shared + ((size_t)min(s0 + u, slabs - 1) * n_tok + t) * H + c, sv[u]);
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (s0 + u < slabs) {
#pragma unroll
                        for (int i = 0; i < VEC; ++i) sh[i] += sv[u][i];
                    }
            }
            const float gt = gate ? gate[t] : 1.f;
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] = fmaf(gt, sh[i], acc[i]);
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = h_old[i] + acc[i];
        if constexpr (VEC == 4) *(float4*)(h + (size_t)t * H + c) = make_float4(v[0], v[1], v[2], v[3]);
        else h[(size_t)t * H + c] = v[0];
    }
    if (!xg) return;
    if (c < H) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) from_float(xg + (size_t)t * H + c + i, v[i] * nw[i]);
    }
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < VEC; ++i) sq = fmaf(v[i], v[i], sq);
    const int n_groups = (H + 255) / 256;
    if constexpr (VEC == 4) {
        const float total = wave_sum(sq);
        const int group = blockIdx.y * 4 + (threadIdx.x >> 6);
        if ((threadIdx.x & 63) == 0 && group < n_groups) ss[t * n_groups + group] = total;
    } else {
        const float total = block_sum<4>(sq, red);
        if (threadIdx.x == 0) ss[t * n_groups + blockIdx.y] = total;
    }
}

// norm_w != nullptr: x_out = round(h * norm_w) of the new rows, in out_dtype, and ss[t][b] = the sum of squares of
// columns [256 b, 256 b + 256) of row t.
FX_API int fx_moe_combine(void* stream, float* h, const float* y, const int* inv, const float* w,
                          const float* shared, const float* gate, int T, int H, int k, int slabs,
                          const void* norm_w, int norm_dtype, void* x_out, int out_dtype, float* ss) {
    FX_REQUIRE(T >= 0 && H > 0 && k > 0 && slabs >= 1, "moe_combine: bad sizes");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    // few rows: a thread per column spreads the row's loads over more waves, which is what counts then
    const bool vec = (long)T * H >= (1L << 18) && H % 4 == 0 && ((uintptr_t)h % 16) == 0 && ((uintptr_t)y % 16) == 0 &&
                     (!shared || ((uintptr_t)shared % 16) == 0);
    const dim3 grid(T, vec ? (H + 1023) / 1024 : (H + 255) / 256);
#define FX_COMBINE(TYPE, XOUT) \
    do { \
        if (vec) moe_combine_kernel<TYPE, 4><<<grid, 256, 0, s>>>(h, y, inv, w, shared, gate, H, k, slabs, norm_w, norm_dtype, XOUT, ss); \
        else moe_combine_kernel<TYPE, 1><<<grid, 256, 0, s>>>(h, y, inv, w, shared, gate, H, k, slabs, norm_w, norm_dtype, XOUT, ss); \
    } while (0)
    if (norm_w) {
        FX_REQUIRE(x_out && ss, "moe_combine: the rows for the norm need places to write");
        FX_REQUIRE(norm_dtype == FX_F32 || norm_dtype == FX_BF16, "moe_combine: unknown norm weight dtype %d", norm_dtype);
        FX_REQUIRE(out_dtype == FX_F32 || out_dtype == FX_BF16, "moe_combine: unknown output dtype %d", out_dtype);
        if (out_dtype == FX_F32) FX_COMBINE(float, (float*)x_out);
        else FX_COMBINE(bf16, (bf16*)x_out);
    } else {
        norm_w = nullptr;
        ss = nullptr;
        FX_COMBINE(float, (float*)nullptr);
    }
#undef FX_COMBINE
    FX_CHECK_LAUNCH("moe_combine");
    return 0;
}

// ---------------------------------------------------------------------------
// h[t, :] += y[t, :] * rsqrt(mean(y[t]^2) + eps) * w: a sublayer's float32 output rows are normed before they
// join the residual stream.  One block per row; two passes over the row (the second finds it in cache).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rmsnorm_add_kernel(float* __restrict__ h, const float* __restrict__ y,
                                                          const void* __restrict__ w, int w_dtype, int H, float eps) {
    __shared__ float red[4];
    const size_t row = (size_t)blockIdx.x * H;
    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += 256) {
        const float v = y[row + c];
        ss = fmaf(v, v, ss);
    }
    ss = block_sum<4>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)H + eps);
    for (int c = threadIdx.x; c < H; c += 256) h[row + c] += y[row + c] * scale * load_as_float(w, w_dtype, c);
}

FX_API int fx_rmsnorm_add(void* stream, float* h, const float* y, const void* w, int w_dtype, int T, int H, float eps) {
    FX_REQUIRE(T >= 0 && H > 0, "rmsnorm_add: bad sizes T=%d H=%d", T, H);
    FX_REQUIRE(w_dtype == FX_F32 || w_dtype == FX_BF16, "rmsnorm_add: unknown weight dtype %d", w_dtype);
    if (T == 0) return 0;
    rmsnorm_add_kernel<<<T, 256, 0, (hipStream_t)stream>>>(h, y, w, w_dtype, H, eps);
    FX_CHECK_LAUNCH("rmsnorm_add");
    return 0;
}

// ---------------------------------------------------------------------------
// The weighted sum of a token's chosen experts where some router outputs are identity experts:
//   out[t, :] = sum_j w[t, j] * (ids[t, j] < E ? y[t*k + j, :] : x[t, :])
// in ascending j; y is float32 [T*k, H] in pair order (rows of identity pairs are read and dropped), x the
// feed-forward's input rows.  With norm_w the sum is then normed and added into the stream,
//   h[t, :] += out[t, :] * rsqrt(mean(out[t]^2) + eps) * norm_w,
// else it is added as it is.  One block per token; `out` [T, H] keeps the sums between the two passes.
// ---------------------------------------------------------------------------
template <typename X, int NW>
__global__ __launch_bounds__(NW * 64) void moe_combine_identity_kernel(float* __restrict__ h, float* __restrict__ out,
                                                                   const float* __restrict__ y, const int* __restrict__ ids,
                                                                   const float* __restrict__ w, const X* __restrict__ x,
                                                                   int E, int H, int k, const void* __restrict__ norm_w,
                                                                   int norm_dtype, float eps) {
    __shared__ float red[NW];
    const int t = blockIdx.x;
    const size_t row = (size_t)t * H;
    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += NW * 64) {
        float acc = 0.f;
        const float xv = to_float(x[row + c]);
        for (int j0 = 0; j0 < k; j0 += 4) {
            // four terms' loads leave together; a row of y is read whatever its pair chose (it is memory of this
            // call's own, written or not) and dropped afterwards, so that no load waits behind a branch
            float yv[4], wv[4];
            int ev[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int j = min(j0 + u, k - 1);
                ev[u] = ids[t * k + j];
                wv[u] = w[t * k + j];
                yv[u] = y[((size_t)t * k + j) * H + c];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (j0 + u < k) acc = fmaf(wv[u], ev[u] < E ? yv[u] : xv, acc);
        }
        out[row + c] = acc;
        ss = fmaf(acc, acc, ss);
    }
    if (!norm_w) {
        for (int c = threadIdx.x; c < H; c += NW * 64) h[row + c] += out[row + c];      // (each thread reads what it wrote)
        return;
    }
    ss = block_sum<NW>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)H + eps);
    for (int c = threadIdx.x; c < H; c += NW * 64) h[row + c] += out[row + c] * scale * load_as_float(norm_w, norm_dtype, c);
}

FX_API int fx_moe_combine_identity(void* stream, float* h, float* out, const float* y, const int* ids, const float* w,
                                   const void* x, int x_dtype, int T, int E, int H, int k, const void* norm_w,
                                   int norm_dtype, float eps) {
    FX_REQUIRE(T >= 0 && H > 0 && k > 0 && E >= 0, "moe_combine_identity: bad sizes");
    FX_REQUIRE(x_dtype == FX_F32 || x_dtype == FX_BF16, "moe_combine_identity: unknown input dtype %d", x_dtype);
    FX_REQUIRE(!norm_w || norm_dtype == FX_F32 || norm_dtype == FX_BF16, "moe_combine_identity: unknown norm weight dtype %d", norm_dtype);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    // wide rows get blocks of 16 waves: every thread then has a column or two, and all of a row's loads are in flight at once
    if (H > 1024) {
        if (x_dtype == FX_F32)
            moe_combine_identity_kernel<float, 16><<<T, 1024, 0, s>>>(h, out, y, ids, w, (const float*)x, E, H, k, norm_w, norm_dtype, eps);
        else
            moe_combine_identity_kernel<bf16, 16><<<T, 1024, 0, s>>>(h, out, y, ids, w, (const bf16*)x, E, H, k, norm_w, norm_dtype, eps);
    } else if (x_dtype == FX_F32)
        moe_combine_identity_kernel<float, 4><<<T, 256, 0, s>>>(h, out, y, ids, w, (const float*)x, E, H, k, norm_w, norm_dtype, eps);
    else
        moe_combine_identity_kernel<bf16, 4><<<T, 256, 0, s>>>(h, out, y, ids, w, (const bf16*)x, E, H, k, norm_w, norm_dtype, eps);
    FX_CHECK_LAUNCH("moe_combine_identity");
    return 0;
}

// ---------------------------------------------------------------------------
// fill a buffer of 32-bit words (used instead of a memset so that callers may
// record it into a HIP graph)
// ---------------------------------------------------------------------------
__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

FX_API int fx_fill_u32(void* stream, void* p, unsigned v, long n) {
    FX_REQUIRE(n >= 0, "fill: bad size");
    if (n == 0) return 0;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 65536) blocks = 65536;
    fill_u32_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((uint32_t*)p, v, (size_t)n);
    FX_CHECK_LAUNCH("fill");
    return 0;
}

// ---------------------------------------------------------------------------
// token ids that are still on the device: tokens[pairs[i][0]] = ids[pairs[i][1]].
// A step whose tokens were sampled by the step before it can be launched before the
// host has read those ids; where it holds one of them, the host wrote a stand-in.
// ---------------------------------------------------------------------------
__global__ void feed_tokens_kernel(int* tokens, const int* ids, const int* pairs, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) tokens[pairs[2 * i]] = ids[pairs[2 * i + 1]];
}

FX_API int fx_feed_tokens(void* stream, int* tokens, const int* ids, const int* pairs, int n) {
    FX_REQUIRE(n >= 0 && tokens && ids && pairs, "feed_tokens: bad arguments");
    if (n == 0) return 0;
    feed_tokens_kernel<<<(n + 255) / 256, 256, 0, (hipStream_t)stream>>>(tokens, ids, pairs, n);
    FX_CHECK_LAUNCH("feed_tokens");
    return 0;
}
