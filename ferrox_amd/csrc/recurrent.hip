// Recurrent mixers: a short causal convolution with its carried inputs, and the gated delta
// rule with one decay per key channel, whose state is a [key channels, value channels] matrix per head.
//
// Everything that enters the recurrence is float32: the convolved q, k, v, the decays, the step
// sizes, the state.  A sequence's tokens lie next to each other in the batch: sequence s owns
// tokens [seq_starts[s], seq_starts[s + 1]); its state lives in slot slots[s] of the state slabs.
#include "common.h"

FX_DEFINE_LAST_ERROR()

// ---------------------------------------------------------------------------
// Short convolution over time per channel:
//   z[t, c] = sum_j taps[c, n-1-j] * x[t-j, c] (+ bias[c]),   j < n
//   y[t, c] = act(z[t, c]) (+ x[t, c] with add_input),   act the identity (0) or silu (1)
// where x[t-j] is a token of this step if it lies in the sequence's portion, else one of the n-1
// inputs carried from before the portion (state[slot, c, :], float32, oldest first; zeros at a sequence's start).
// x and y are float32 or bfloat16 rows; the sums are float32.
// One thread per (four tokens that follow each other in the batch, channel).
// ---------------------------------------------------------------------------
#define CONV_MAX_TAPS 16
#define CONV_TOKENS 4        // tokens to a thread: neighbouring tokens share all but one of their inputs
__device__ __forceinline__ float conv_finish(float acc, const void* bias, int taps_dtype, int c, int act, int add_input, float x_now) {
    if (bias) acc += load_as_float(bias, taps_dtype, c);
    if (act) acc = acc / (1.0f + expf(-acc));
    return add_input ? acc + x_now : acc;
}

template <int TAPS, typename TX, typename TY>          // TAPS: the number of taps where it is 2..4 (the inputs then live in registers), else 0
__global__ __launch_bounds__(256) void short_conv_kernel(const TX* __restrict__ x, long ldx, TY* __restrict__ y, long ldy,
                                                         const void* __restrict__ taps, int taps_dtype, int n_taps,
                                                         const float* __restrict__ state, const int* __restrict__ token_seq,
                                                         const int* __restrict__ seq_starts, const int* __restrict__ slots,
                                                         int n_tokens, int C, const void* __restrict__ bias, int act, int add_input) {
    const int t0 = blockIdx.y * CONV_TOKENS;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    if constexpr (TAPS > 0) {
        // the inputs of tokens t0 - TAPS + 1 .. t0 + 3 once, then every token of the four takes its own from them (those
        // of its sequence's portion) or from what its sequence carried
        float w[TAPS], xin[CONV_TOKENS + TAPS - 1];
#pragma unroll
        for (int j = 0; j < TAPS; ++j) w[j] = load_as_float(taps, taps_dtype, (size_t)c * TAPS + j);
#pragma unroll
        for (int e = 0; e < CONV_TOKENS + TAPS - 1; ++e) {
            const int t = t0 - (TAPS - 1) + e;
            xin[e] = (t >= 0 && t < n_tokens) ? to_float(x[(size_t)t * ldx + c]) : 0.f;
        }
#pragma unroll
        for (int u = 0; u < CONV_TOKENS; ++u) {
            const int t = t0 + u;
            if (t >= n_tokens) break;
            const int s = token_seq[t];
            const int i = t - seq_starts[s];             // place in the portion
            const float* carried = state + ((size_t)slots[s] * C + c) * (TAPS - 1);
            float acc = 0.f;
#pragma unroll
            for (int j = TAPS - 1; j >= 0; --j) {        // oldest input first
                const float xv = j <= i ? xin[u + TAPS - 1 - j] : carried[TAPS - 1 + i - j];
                acc = fmaf(w[TAPS - 1 - j], xv, acc);
            }
            from_float(y + (size_t)t * ldy + c, conv_finish(acc, bias, taps_dtype, c, act, add_input, xin[u + TAPS - 1]));
        }
    } else {
        for (int t = t0; t < min(t0 + CONV_TOKENS, n_tokens); ++t) {
            const int s = token_seq[t];
            const int i = t - seq_starts[s];
            const float* carried = state + ((size_t)slots[s] * C + c) * (n_taps - 1);
            float acc = 0.f;
            for (int j = n_taps - 1; j >= 0; --j) {
                const float xv = j <= i ? to_float(x[(size_t)(t - j) * ldx + c]) : carried[n_taps - 1 + i - j];
                acc = fmaf(load_as_float(taps, taps_dtype, (size_t)c * n_taps + n_taps - 1 - j), xv, acc);
            }
            from_float(y + (size_t)t * ldy + c, conv_finish(acc, bias, taps_dtype, c, act, add_input, to_float(x[(size_t)t * ldx + c])));
        }
    }
}

// After the step: the last n-1 inputs of every sequence, oldest first.  One thread per (sequence, channel);
// it reads an entry that it is about to overwrite before it writes it (entries move toward the front).
template <typename TX>
__global__ __launch_bounds__(256) void conv_carry_kernel(const TX* __restrict__ x, long ldx, float* __restrict__ state,
                                                         const int* __restrict__ seq_starts, const int* __restrict__ slots,
                                                         int C, int n_taps) {
    const int s = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int t0 = seq_starts[s], n = seq_starts[s + 1] - t0;
    if (n <= 0) return;
    float* carried = state + ((size_t)slots[s] * C + c) * (n_taps - 1);
    for (int j = 0; j < n_taps - 1; ++j) {
        const int i = n - (n_taps - 1) + j;          // place in the portion of the input that entry j holds afterwards
        carried[j] = i >= 0 ? to_float(x[(size_t)(t0 + i) * ldx + c]) : carried[j + n];
    }
}

template <typename TX, typename TY>
static void launch_short_conv(hipStream_t s, const void* x, long ldx, void* y, long ldy, const void* taps, int taps_dtype,
                              int n_taps, float* state, const int* token_seq, const int* seq_starts, const int* slots,
                              int T, int n_seqs, int C, const void* bias, int act, int add_input) {
    const dim3 grid((C + 255) / 256, (T + CONV_TOKENS - 1) / CONV_TOKENS);
#define FX_CONV(TAPS_) short_conv_kernel<TAPS_, TX, TY><<<grid, 256, 0, s>>>((const TX*)x, ldx, (TY*)y, ldy, taps, taps_dtype, n_taps, state, token_seq, seq_starts, slots, T, C, bias, act, add_input)
    if (n_taps == 4) FX_CONV(4);
    else if (n_taps == 3) FX_CONV(3);
    else if (n_taps == 2) FX_CONV(2);
    else FX_CONV(0);
#undef FX_CONV
    if (n_taps > 1)
        conv_carry_kernel<TX><<<dim3((C + 255) / 256, n_seqs), 256, 0, s>>>((const TX*)x, ldx, state, seq_starts, slots, C, n_taps);
}

FX_API int fx_short_conv(void* stream, const void* x, int x_dtype, long ldx, void* y, int y_dtype, long ldy, const void* taps,
                         int taps_dtype, int n_taps, float* state, const int* token_seq, const int* seq_starts, const int* slots,
                         int T, int n_seqs, int C, const void* bias, int act, int add_input) {
    FX_REQUIRE(T >= 0 && n_seqs >= 0 && C > 0, "short_conv: bad sizes T=%d sequences=%d C=%d", T, n_seqs, C);
    FX_REQUIRE(n_taps >= 1 && n_taps <= CONV_MAX_TAPS, "short_conv: %d taps, this kernel takes 1..%d", n_taps, CONV_MAX_TAPS);
    FX_REQUIRE(ldx >= C && ldy >= C, "short_conv: rows of %ld and %ld hold fewer than %d channels", ldx, ldy, C);
    FX_REQUIRE(taps_dtype == FX_F32 || taps_dtype == FX_BF16, "short_conv: unknown dtype %d of the taps", taps_dtype);
    FX_REQUIRE((x_dtype == FX_F32 || x_dtype == FX_BF16) && (y_dtype == FX_F32 || y_dtype == x_dtype), "short_conv: rows of type %d into rows of type %d", x_dtype, y_dtype);
    FX_REQUIRE(act == 0 || act == 1, "short_conv: activation %d (0 none, 1 silu)", act);
    FX_REQUIRE(T <= 4 * 65535 && n_seqs <= 65535, "short_conv: %d tokens of %d sequences are more than a launch takes", T, n_seqs);
    FX_REQUIRE(x != y, "short_conv: the output must not be the input (carried inputs are read from it afterwards)");
    if (T == 0 || n_seqs == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
#define FX_ARGS s, x, ldx, y, ldy, taps, taps_dtype, n_taps, state, token_seq, seq_starts, slots, T, n_seqs, C, bias, act, add_input
    if (x_dtype == FX_F32) launch_short_conv<float, float>(FX_ARGS);
    else if (y_dtype == FX_F32) launch_short_conv<bf16, float>(FX_ARGS);
    else launch_short_conv<bf16, bf16>(FX_ARGS);
#undef FX_ARGS
    FX_CHECK_LAUNCH("short_conv");
    return 0;
}

// ---------------------------------------------------------------------------
// What the delta rule's recurrence reads, made per token from the convolved q and k and from the
// projections of the gates (all float32):
//   qn = q / sqrt(sum(q^2) + 1e-6) * D^-1/2,  kn = k / sqrt(sum(k^2) + 1e-6)        per q/k head
//   decay[h, i] = exp(-exp(A_log[h]) * softplus(a[h, i] + dt_bias[h, i]))             per head and key channel
//                 (per_head: a and dt_bias hold one number a head, a[h] and dt_bias[h], and all D channels of a
//                 head receive the same decay)
//   beta[h] = sigmoid(b[h])
//   kq[g] = kn[g] . qn[g]                                                             per q/k head (the recurrence needs it per token)
// Blocks (token, part): part p makes 256 of the token's decays and, a wave each, heads 4p .. 4p+3 of q and k (a
// decode step's few tokens then still spread over many blocks).
// ---------------------------------------------------------------------------
__device__ __forceinline__ float softplus_f(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

__global__ __launch_bounds__(256) void delta_prepare_kernel(const float* __restrict__ q, long ldq, const float* __restrict__ k, long ldk,
                                                            const float* __restrict__ a, long lda, const float* __restrict__ b, long ldb,
                                                            const void* __restrict__ A_log, const void* __restrict__ dt_bias, int w_dtype,
                                                            float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ decay,
                                                            float* __restrict__ beta, float* __restrict__ kq, int H, int G, int D,
                                                            int per_head) {
    const int t = blockIdx.x, part = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int g = part * 4 + wave; g < G; g += 4 * gridDim.y) {          // a wave per head of q and k
        const float* qs = q + (size_t)t * ldq + (size_t)g * D;
        const float* ks = k + (size_t)t * ldk + (size_t)g * D;
        float sq = 0.f, sk = 0.f;
        for (int i = lane; i < D; i += 64) {
            sq = fmaf(qs[i], qs[i], sq);
            sk = fmaf(ks[i], ks[i], sk);
        }
        const float q_scale = 1.0f / sqrtf(wave_sum(sq) + 1e-6f) * (1.0f / sqrtf((float)D));
        const float k_scale = 1.0f / sqrtf(wave_sum(sk) + 1e-6f);
        float dot = 0.f;
        for (int i = lane; i < D; i += 64) {
            const float qv = qs[i] * q_scale, kv = ks[i] * k_scale;
            qn[((size_t)t * G + g) * D + i] = qv;
            kn[((size_t)t * G + g) * D + i] = kv;
            dot = fmaf(kv, qv, dot);
        }
        dot = wave_sum(dot);
        if (lane == 0) kq[(size_t)t * G + g] = dot;
    }
    for (int idx = part * 256 + threadIdx.x; idx < H * D; idx += 256 * gridDim.y) {
        const int h = idx / D, src = per_head ? h : idx;
        const float rate = expf(load_as_float(A_log, w_dtype, h));
        const float step = softplus_f(a[(size_t)t * lda + src] + load_as_float(dt_bias, w_dtype, src));
        decay[(size_t)t * H * D + idx] = expf(-rate * step);
    }
    if (part == 0)
        for (int h = threadIdx.x; h < H; h += 256) beta[(size_t)t * H + h] = 1.0f / (1.0f + expf(-b[(size_t)t * ldb + h]));
}

FX_API int fx_delta_prepare(void* stream, const float* q, long ldq, const float* k, long ldk, const float* a, long lda,
                            const float* b, long ldb, const void* A_log, const void* dt_bias, int w_dtype, float* qn,
                            float* kn, float* decay, float* beta, float* kq, int T, int H, int G, int D, int per_head) {
    FX_REQUIRE(T >= 0 && H > 0 && G > 0 && D > 0 && H % G == 0, "delta_prepare: bad sizes T=%d H=%d G=%d D=%d", T, H, G, D);
    FX_REQUIRE(w_dtype == FX_F32 || w_dtype == FX_BF16, "delta_prepare: unknown dtype %d", w_dtype);
    if (T == 0) return 0;
    const int parts = (int)fminl(1024, fmaxl((H * (long)D + 255) / 256, (G + 3) / 4));
    delta_prepare_kernel<<<dim3(T, parts), 256, 0, (hipStream_t)stream>>>(q, ldq, k, ldk, a, lda, b, ldb, A_log, dt_bias, w_dtype, qn, kn,
                                                             decay, beta, kq, H, G, D, per_head);
    FX_CHECK_LAUNCH("delta_prepare");
    return 0;
}

// ---------------------------------------------------------------------------
// Two small float32 products of few rows in one launch: out_i[t, n] = sum_k x_i[t, k] * wt_i[k, n], i = 0, 1, k
// ascending in one accumulator (the sums of the float32 product kernel, so a row gets the same bits from either).
// These are the second halves of the delta rule's two low-rank projections (decay and output gate): K is the
// inner size (tens to a few hundred), the weights are kept transposed [K, N] so that neighbouring lanes read
// neighbouring columns, and a decode step's few rows make them two launches' worth of waiting otherwise.
// Grid: (ceil(max N / 256), rows, 2).
// ---------------------------------------------------------------------------
#define PAIR_MAX_K 512
__global__ __launch_bounds__(256) void small_rows_pair_kernel(const float* __restrict__ x0, long ldx0, const float* __restrict__ wt0,
                                                              float* __restrict__ out0, long ldo0, int K0, int N0,
                                                              const float* __restrict__ x1, long ldx1, const float* __restrict__ wt1,
                                                              float* __restrict__ out1, long ldo1, int K1, int N1) {
    __shared__ float xs[PAIR_MAX_K];
    const bool second = blockIdx.z == 1;
    const float* x = second ? x1 : x0;
    const float* wt = second ? wt1 : wt0;
    float* out = second ? out1 : out0;
    const long ldx = second ? ldx1 : ldx0, ldo = second ? ldo1 : ldo0;
    const int K = second ? K1 : K0, N = second ? N1 : N0;
    const int t = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
    if (blockIdx.x * 256 >= N) return;               // (the same in every thread of the block)
    for (int k = threadIdx.x; k < K; k += 256) xs[k] = x[(size_t)t * ldx + k];
    __syncthreads();
    if (n >= N) return;
    float acc = 0.f;
#pragma unroll 8
    for (int k = 0; k < K; ++k) acc = fmaf(xs[k], wt[(size_t)k * N + n], acc);
    out[(size_t)t * ldo + n] = acc;
}

FX_API int fx_small_rows_pair(void* stream, const float* x0, long ldx0, const float* wt0, float* out0, long ldo0, int K0, int N0,
                              const float* x1, long ldx1, const float* wt1, float* out1, long ldo1, int K1, int N1, int T) {
    FX_REQUIRE(T >= 0 && T <= 65535, "small_rows_pair: %d rows", T);
    FX_REQUIRE(K0 >= 1 && K0 <= PAIR_MAX_K && K1 >= 1 && K1 <= PAIR_MAX_K, "small_rows_pair: inner sizes %d and %d, this kernel takes 1..%d", K0, K1, PAIR_MAX_K);
    FX_REQUIRE(N0 >= 1 && N1 >= 1 && ldx0 >= K0 && ldx1 >= K1 && ldo0 >= N0 && ldo1 >= N1, "small_rows_pair: bad sizes");
    if (T == 0) return 0;
    const int widest = N0 > N1 ? N0 : N1;
    small_rows_pair_kernel<<<dim3((widest + 255) / 256, T, 2), 256, 0, (hipStream_t)stream>>>(x0, ldx0, wt0, out0, ldo0, K0, N0,
                                                                                               x1, ldx1, wt1, out1, ldo1, K1, N1);
    FX_CHECK_LAUNCH("small_rows_pair");
    return 0;
}

// ---------------------------------------------------------------------------
// A block-diagonal float32 product of few rows in one launch: the K-wide part j of row t, times the transposed matrix
// wt[j] [K, N] of that part, out[t, j, n] = sum_k x[t, j K + k] * wt[j, k, n], k ascending in one accumulator.  These
// are the gates of a recurrent unit whose channels are cut into parts with a square matrix each; a decode step's few
// rows would wait in a tiled product's launch for nothing.  Grid: (ceil(N / 256), rows, parts).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void small_rows_parts_kernel(const float* __restrict__ x, long ldx, const float* __restrict__ wt,
                                                               float* __restrict__ out, int K, int N, int parts) {
    __shared__ float xs[PAIR_MAX_K];
    const int t = blockIdx.y, j = blockIdx.z, n = blockIdx.x * 256 + threadIdx.x;
    for (int k = threadIdx.x; k < K; k += 256) xs[k] = x[(size_t)t * ldx + (size_t)j * K + k];
    __syncthreads();
    if (n >= N) return;
    const float* w = wt + (size_t)j * K * N;
    float acc = 0.f;
#pragma unroll 8
    for (int k = 0; k < K; ++k) acc = fmaf(xs[k], w[(size_t)k * N + n], acc);
    out[((size_t)t * parts + j) * N + n] = acc;
}

FX_API int fx_small_rows_parts(void* stream, const float* x, long ldx, const float* wt, float* out, int K, int N, int parts, int T) {
    FX_REQUIRE(T >= 0 && T <= 65535 && parts >= 1 && parts <= 65535, "small_rows_parts: %d rows of %d parts", T, parts);
    FX_REQUIRE(K >= 1 && K <= PAIR_MAX_K && N >= 1 && ldx >= (long)parts * K, "small_rows_parts: parts of %d columns (up to %d) in rows of %ld", K, PAIR_MAX_K, ldx);
    if (T == 0) return 0;
    small_rows_parts_kernel<<<dim3((N + 255) / 256, T, parts), 256, 0, (hipStream_t)stream>>>(x, ldx, wt, out, K, N, parts);
    FX_CHECK_LAUNCH("small_rows_parts");
    return 0;
}

// ---------------------------------------------------------------------------
// The recurrence.  Per head, with S [D, V] carried from token to token:
//   S <- diag(decay_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
// Tokens follow each other; columns of S never meet.  A wave owns 64 / LPC columns, LPC = 16 or 32 lanes to a
// column: lane (c, r), c = lane / LPC, r = lane % LPC, holds rows [r DR, (r + 1) DR) of its column in registers
// (LPC DR >= D; rows past D stay zero).  Per token it forms, over its rows, the parts of (dS)^T k and (dS)^T q
// (k.q comes with the token, from the kernel above); the lanes of a column add theirs with four rotations inside their row of 16 lanes and, for 32 lanes, one
// exchange between neighbouring rows (every lane gets the same bits: each step adds two sums of complementary
// lanes, and a + b is b + a); then u and o = (dS)^T q + u (k.q) follow, and S takes k u^T.
// A token's k, q and decay are the same for every column of a head, and reading them is most of the traffic: a
// block of NW waves (NW 64 / LPC columns) brings them into LDS once for all its waves, a group of P tokens at a
// time and a group ahead (memory is waited for once a group, not once a token; one barrier a group), and lanes
// of one r read their rows as broadcasts.  (A wave that fetched for itself made a layer read 3 GB for a prompt of
// 2,048 tokens at 16 heads of 128 x 128, and more waves made it slower.)
// The state is kept transposed, [slot][head][V][D]: a lane's rows of its column lie next to each other, and a
// wave reads and writes contiguous floats (a decode step is little more than that read and write).
// VEC: D is a multiple of 4, and rows travel in 16-byte pieces.  Grid: (ceil(V / (NW 64 / LPC)), heads, sequences).
// ---------------------------------------------------------------------------
template <int LPC>
__device__ __forceinline__ float column_sum(float v) {      // over the LPC lanes of a column, in each of them
    v += row_rotated<0x128>(v);      // row_ror:8
    v += row_rotated<0x124>(v);      // row_ror:4
    v += row_rotated<0x122>(v);      // row_ror:2
    v += row_rotated<0x121>(v);      // row_ror:1
    if constexpr (LPC == 32) {
        float o;
        v = wave_partner_16(v, o) + o;      // rows 0 and 1, rows 2 and 3
    }
    return v;
}

template <int DR, int LPC, bool VEC, int NW>
__global__ __launch_bounds__(NW * 64) void channel_delta_kernel(const float* __restrict__ qn, const float* __restrict__ kn,
                                                                const float* __restrict__ decay, const float* __restrict__ beta,
                                                                const float* __restrict__ kq_all, const float* __restrict__ v, long ldv, float* __restrict__ out, long ldo,
                                                                float* __restrict__ state, const int* __restrict__ seq_starts,
                                                                const int* __restrict__ slots, int H, int G, int D, int V) {
    constexpr int DP = LPC * DR;                     // rows as a wave holds them
    constexpr int W = VEC ? 4 : 1;                   // floats per load
    constexpr int P = 8;                             // tokens that travel together
    constexpr int NT = NW * 64;
    constexpr int PIECES = 3 * DP / W;               // loads that bring one token's (k | q | decay)
    constexpr int NL = (P * PIECES + NT - 1) / NT;   // loads a thread makes per group
    constexpr int COLS = 64 / LPC;
    static_assert(DR % 4 == 0, "a lane's rows are read from LDS in 16-byte pieces");
    __shared__ __attribute__((aligned(16))) float kqd[2][P][3][DP];      // two groups of P tokens x (k, q, decay)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane % LPC, j = (blockIdx.x * NW + wave) * COLS + lane / LPC;
    const int h = blockIdx.y, s = blockIdx.z, g = h / (H / G);
    const int t0 = seq_starts[s], t1 = seq_starts[s + 1];
    if (t1 <= t0) return;                            // (the same in every thread of the block)
    const bool col = j < V;
    float* S_g = state + (((size_t)slots[s] * H + h) * V + (col ? j : 0)) * D + r * DR;
    float S[DR];
#pragma unroll
    for (int i = 0; i < DR; i += 4) {
        if constexpr (VEC) {
            const bool in = col && r * DR + i < D;      // (D % 4 == 0: a piece is inside or outside as a whole)
            const float4 x = in ? *(const float4*)(S_g + i) : make_float4(0.f, 0.f, 0.f, 0.f);
            S[i] = x.x; S[i + 1] = x.y; S[i + 2] = x.z; S[i + 3] = x.w;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) S[i + e] = (col && r * DR + i + e < D) ? S_g[i + e] : 0.f;
        }
    }
    // a group's operands: piece number idx = n NT + tid of the group's P PIECES goes to kqd[.] at idx W, which is
    // token idx / PIECES, then k, q or decay, then the row; pieces past D, past the group or past the sequence are zeros
    float nxt[NL][W], v_nxt[P], b_nxt[P], kq_nxt[P];
    auto fetch = [&](int first) {
#pragma unroll
        for (int n = 0; n < NL; ++n) {
            const int idx = n * NT + tid, p = idx / PIECES, e = (idx - p * PIECES) * W, which = e / DP, row = e - which * DP;
            const int t = first + p;
            const bool ok = idx < P * PIECES && t < t1 && row < D;
            const float* src = which == 0 ? kn + ((size_t)t * G + g) * D : (which == 1 ? qn + ((size_t)t * G + g) * D
                                                                                         : decay + ((size_t)t * H + h) * D);
            if constexpr (VEC) {
                const float4 x = ok ? *(const float4*)(src + row) : make_float4(0.f, 0.f, 0.f, 0.f);
                nxt[n][0] = x.x; nxt[n][W - 3] = x.y; nxt[n][W - 2] = x.z; nxt[n][W - 1] = x.w;
            } else {
                nxt[n][0] = ok ? src[row] : 0.f;
            }
        }
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const bool live = first + p < t1;
            v_nxt[p] = (live && col) ? v[(size_t)(first + p) * ldv + (size_t)h * V + j] : 0.f;
            b_nxt[p] = live ? beta[(size_t)(first + p) * H + h] : 0.f;
            kq_nxt[p] = live ? kq_all[(size_t)(first + p) * G + g] : 0.f;
        }
    };
    auto stage = [&](int slot) {
#pragma unroll
        for (int n = 0; n < NL; ++n) {
            const int idx = n * NT + tid;
            if (idx < P * PIECES) {
                float* dst = &kqd[slot][0][0][0] + (size_t)idx * W;
                if constexpr (VEC) *(float4*)dst = make_float4(nxt[n][0], nxt[n][W - 3], nxt[n][W - 2], nxt[n][W - 1]);
                else *dst = nxt[n][0];
            }
        }
    };
    fetch(t0);
    stage(0);
    __syncthreads();
    for (int first = t0, cur = 0; first < t1; first += P, cur ^= 1) {
        float v_cur[P], b_cur[P], kq_cur[P];
#pragma unroll
        for (int p = 0; p < P; ++p) {
            v_cur[p] = v_nxt[p];
            b_cur[p] = b_nxt[p];
            kq_cur[p] = kq_nxt[p];
        }
        const bool more = first + P < t1;
        if (more) fetch(first + P);                  // the next group's operands leave now and are staged after this group's work
        auto token = [&](int p, int t) {
            const float* kk = &kqd[cur][p][0][r * DR];
            const float* qq = &kqd[cur][p][1][r * DR];
            const float* dd = &kqd[cur][p][2][r * DR];
            float kv[DR];
            float sk = 0.f, sq = 0.f;
#pragma unroll
            for (int i = 0; i < DR; i += 4) {
                const float4 k4 = *(const float4*)(kk + i), q4 = *(const float4*)(qq + i), d4 = *(const float4*)(dd + i);
                const float ka[4] = {k4.x, k4.y, k4.z, k4.w}, qa[4] = {q4.x, q4.y, q4.z, q4.w}, da[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    S[i + e] *= da[e];
                    sk = fmaf(S[i + e], ka[e], sk);
                    sq = fmaf(S[i + e], qa[e], sq);
                    kv[i + e] = ka[e];
                }
            }
            sk = column_sum<LPC>(sk);
            sq = column_sum<LPC>(sq);
            const float u = b_cur[p] * (v_cur[p] - sk);
            if (col && r == 0) out[(size_t)t * ldo + (size_t)h * V + j] = fmaf(u, kq_cur[p], sq);
#pragma unroll
            for (int i = 0; i < DR; ++i) S[i] = fmaf(kv[i], u, S[i]);
        };
        if (first + P <= t1) {                       // a whole group: one stretch of code, so that a token's LDS reads leave
#pragma unroll                                       // while the token before it is worked on
            for (int p = 0; p < P; ++p) token(p, first + p);
        } else {
#pragma unroll
            for (int p = 0; p < P; ++p)
                if (first + p < t1) token(p, first + p);
        }
        if (more) stage(cur ^ 1);                    // (the buffer that every wave left before the last barrier)
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < DR; i += 4) {
        if constexpr (VEC) {
            if (col && r * DR + i < D) *(float4*)(S_g + i) = make_float4(S[i], S[i + 1], S[i + 2], S[i + 3]);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (col && r * DR + i + e < D) S_g[i + e] = S[i + e];
        }
    }
}

FX_API int fx_channel_delta(void* stream, const float* qn, const float* kn, const float* decay, const float* beta,
                            const float* kq, const float* v, long ldv, float* out, long ldo, float* state, const int* seq_starts,
                            const int* slots, int n_seqs, int H, int G, int D, int V) {
    FX_REQUIRE(n_seqs >= 0 && H > 0 && G > 0 && H % G == 0, "channel_delta: bad sizes sequences=%d H=%d G=%d", n_seqs, H, G);
    FX_REQUIRE(D >= 1 && D <= 256 && V >= 1, "channel_delta: key size %d (up to 256) and value size %d", D, V);
    FX_REQUIRE(ldv >= (long)H * V && ldo >= (long)H * V, "channel_delta: rows of %ld and %ld hold fewer than %d values", ldv, ldo, H * V);
    FX_REQUIRE(n_seqs <= 65535 && H <= 65535, "channel_delta: %d sequences of %d heads are more than a launch takes", n_seqs, H);
    if (n_seqs == 0) return 0;
    const bool vec = D % 4 == 0 && (((uintptr_t)state | (uintptr_t)qn | (uintptr_t)kn | (uintptr_t)decay) % 16) == 0;
    hipStream_t s = (hipStream_t)stream;
#define FX_DELTA(DR_, LPC_, NW_)                                                                                              \
    do {                                                                                                                      \
        const int per_block = NW_ * 64 / LPC_;                                                                                \
        const dim3 grid((V + per_block - 1) / per_block, H, n_seqs);                                                          \
        if (vec) channel_delta_kernel<DR_, LPC_, true, NW_><<<grid, NW_ * 64, 0, s>>>(qn, kn, decay, beta, kq, v, ldv, out, ldo, state, seq_starts, slots, H, G, D, V); \
        else channel_delta_kernel<DR_, LPC_, false, NW_><<<grid, NW_ * 64, 0, s>>>(qn, kn, decay, beta, kq, v, ldv, out, ldo, state, seq_starts, slots, H, G, D, V);    \
    } while (0)
    // (blocks of 8 or 16 columns: with fewer waves to a block a block's fetch is shared by fewer, with more the
    // waves of one CU read the same operands out of its LDS more often; four waves measured best at 16 heads of
    // 128 x 128, 4.65 against 4.78 ms for four layers of a 2,048-token prompt with eight)
    if (D <= 64 && V <= 32) FX_DELTA(4, 16, 2);
    else if (D <= 64) FX_DELTA(4, 16, 4);
    else if (D <= 128) FX_DELTA(4, 32, 4);
    else FX_DELTA(8, 32, 8);
#undef FX_DELTA
    FX_CHECK_LAUNCH("channel_delta");
    return 0;
}

// ---------------------------------------------------------------------------
// The read-out's way to the output projection: every head's o is divided by its root mean square over V
// (eps inside the root), times a weight (w_stride 0: one [V] shared by the heads; w_stride V: [H, V], a weight per
// head and channel), times sigmoid(gate[h, :]) (gate_act 0) or silu(gate[h, :]) (gate_act 1).  With `nq` and `m`
// (float32 [T, H] each) the head's o is first divided by max(|nq|, exp(-m)) + 1e-6: the normaliser of a matrix memory
// whose gates are kept in range by a running maximum m.  One wave per (token, head).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gated_head_norm_kernel(const float* __restrict__ o, long ldo, const float* __restrict__ gate,
                                                              long ldg, const void* __restrict__ w, int w_dtype, int w_stride, T* __restrict__ y,
                                                              long ldy, int n_rows, int H, int V, float eps, int gate_act,
                                                              const float* __restrict__ nq, const float* __restrict__ m) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= n_rows) return;
    const int t = row / H, h = row - t * H;
    const float* src = o + (size_t)t * ldo + (size_t)h * V;
    float inv_den = 1.0f;
    if (nq) inv_den = 1.0f / (fmaxf(fabsf(nq[row]), expf(-m[row])) + 1e-6f);
    float ss = 0.f;
    for (int i = lane; i < V; i += 64) {
        const float x = src[i] * inv_den;
        ss = fmaf(x, x, ss);
    }
    ss = wave_sum(ss);
    const float scale = 1.0f / sqrtf(ss / (float)V + eps);
    for (int i = lane; i < V; i += 64) {
        const float gx = gate[(size_t)t * ldg + (size_t)h * V + i];
        const float gt = (gate_act ? gx : 1.0f) / (1.0f + expf(-gx));
        from_float(y + (size_t)t * ldy + (size_t)h * V + i, src[i] * inv_den * scale * load_as_float(w, w_dtype, (size_t)h * w_stride + i) * gt);
    }
}

// The same for long rows (all heads normed as one row of thousands of channels): a block per (token, head), so that a
// decode step's few rows are not one wave's long loop each.
template <typename T>
__global__ __launch_bounds__(256) void gated_row_norm_kernel(const float* __restrict__ o, long ldo, const float* __restrict__ gate,
                                                             long ldg, const void* __restrict__ w, int w_dtype, int w_stride, T* __restrict__ y,
                                                             long ldy, int H, int V, float eps, int gate_act,
                                                             const float* __restrict__ nq, const float* __restrict__ m) {
    __shared__ float red[4];
    const int row = blockIdx.x, t = row / H, h = row - t * H;
    const float* src = o + (size_t)t * ldo + (size_t)h * V;
    float inv_den = 1.0f;
    if (nq) inv_den = 1.0f / (fmaxf(fabsf(nq[row]), expf(-m[row])) + 1e-6f);
    float ss = 0.f;
    for (int i = threadIdx.x; i < V; i += 256) {
        const float x = src[i] * inv_den;
        ss = fmaf(x, x, ss);
    }
    ss = block_sum<4>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)V + eps);
    for (int i = threadIdx.x; i < V; i += 256) {
        const float gx = gate[(size_t)t * ldg + (size_t)h * V + i];
        const float gt = (gate_act ? gx : 1.0f) / (1.0f + expf(-gx));
        from_float(y + (size_t)t * ldy + (size_t)h * V + i, src[i] * inv_den * scale * load_as_float(w, w_dtype, (size_t)h * w_stride + i) * gt);
    }
}

FX_API int fx_gated_head_norm(void* stream, int out_dtype, const float* o, long ldo, const float* gate, long ldg,
                              const void* w, int w_dtype, int w_per_head, void* y, long ldy, int T, int H, int V, float eps,
                              int gate_act, const float* nq, const float* m) {
    FX_REQUIRE(gate_act == 0 || gate_act == 1, "gated_head_norm: gate activation %d (0 sigmoid, 1 silu)", gate_act);
    FX_REQUIRE(T >= 0 && H > 0 && V > 0, "gated_head_norm: bad sizes T=%d H=%d V=%d", T, H, V);
    FX_REQUIRE(w_dtype == FX_F32 || w_dtype == FX_BF16, "gated_head_norm: unknown weight dtype %d", w_dtype);
    FX_REQUIRE((long)T * H < (1L << 31), "gated_head_norm: too many rows for one launch");
    FX_REQUIRE((nq == nullptr) == (m == nullptr), "gated_head_norm: the normaliser's product and the running maximum come together");
    if (T == 0) return 0;
    const int rows = T * H, ws = w_per_head ? V : 0;
    hipStream_t s = (hipStream_t)stream;
    if (V > 512 && (out_dtype == FX_F32 || out_dtype == FX_BF16)) {
        if (out_dtype == FX_F32) gated_row_norm_kernel<float><<<rows, 256, 0, s>>>(o, ldo, gate, ldg, w, w_dtype, ws, (float*)y, ldy, H, V, eps, gate_act, nq, m);
        else gated_row_norm_kernel<bf16><<<rows, 256, 0, s>>>(o, ldo, gate, ldg, w, w_dtype, ws, (bf16*)y, ldy, H, V, eps, gate_act, nq, m);
        FX_CHECK_LAUNCH("gated_head_norm");
        return 0;
    }
    if (out_dtype == FX_F32)
        gated_head_norm_kernel<float><<<(rows + 3) / 4, 256, 0, s>>>(o, ldo, gate, ldg, w, w_dtype, ws, (float*)y, ldy, rows, H, V, eps, gate_act, nq, m);
    else if (out_dtype == FX_BF16)
        gated_head_norm_kernel<bf16><<<(rows + 3) / 4, 256, 0, s>>>(o, ldo, gate, ldg, w, w_dtype, ws, (bf16*)y, ldy, rows, H, V, eps, gate_act, nq, m);
    else
        return fx_fail("gated_head_norm: unknown output dtype %d", out_dtype);
    FX_CHECK_LAUNCH("gated_head_norm");
    return 0;
}

// ---------------------------------------------------------------------------
// A matrix memory with one forgetting factor and one writing factor per head and token (linear attention with a
// decay; the matrix memory of an LSTM with exponential gates):
//   S <- keep_t S + take_t k_t v_t^T;   o_t = q_scale S^T q_t           S: [D, V] per head, float32
// keep [T, H] (or, with keep_const, [H]: the same factor at every token) and take [T, H] (null: 1) are float32.
// With `normalizer`, the state has one more column, n <- keep_t n + take_t k_t, and nq[t, h] = q_scale n_t . q_t
// leaves beside o: it is column V of a state [slot][head][V + 1][D], computed as a column whose value is always 1.
// Lanes, columns, the state's transposed layout, the groups of P tokens that a block of waves brings into LDS a
// group ahead: as in the delta rule's kernel above; a token's work is one pass over the lane's rows (S updated,
// then its part of S^T q) and one sum over the lanes of a column.
// Grid: (ceil((V + normalizer) / (NW 64 / LPC)), heads, sequences).
// ---------------------------------------------------------------------------
template <int DR, int LPC, bool VEC, int NW>
__global__ __launch_bounds__(NW * 64) void gated_outer_kernel(const float* __restrict__ q, long ldq, const float* __restrict__ k, long ldk,
                                                              const float* __restrict__ v, long ldv, const float* __restrict__ keep,
                                                              int keep_const, const float* __restrict__ take, float* __restrict__ out,
                                                              long ldo, float* __restrict__ nq, float* __restrict__ state,
                                                              const int* __restrict__ seq_starts, const int* __restrict__ slots,
                                                              int H, int G, int D, int V, int VS, float q_scale) {
    constexpr int DP = LPC * DR;                     // rows as a wave holds them
    constexpr int W = VEC ? 4 : 1;                   // floats per load
    constexpr int P = 8;                             // tokens that travel together
    constexpr int NT = NW * 64;
    constexpr int PIECES = 2 * DP / W;               // loads that bring one token's (k | q)
    constexpr int NL = (P * PIECES + NT - 1) / NT;   // loads a thread makes per group
    constexpr int COLS = 64 / LPC;
    static_assert(DR % 4 == 0, "a lane's rows are read from LDS in 16-byte pieces");
    __shared__ __attribute__((aligned(16))) float kq[2][P][2][DP];      // two groups of P tokens x (k, q)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane % LPC, j = (blockIdx.x * NW + wave) * COLS + lane / LPC;
    const int h = blockIdx.y, s = blockIdx.z, g = h / (H / G);
    const int t0 = seq_starts[s], t1 = seq_starts[s + 1];
    if (t1 <= t0) return;                            // (the same in every thread of the block)
    const bool col = j < VS, ones = j == V;          // VS = V (+ 1: the normaliser's column, whose value is 1)
    float* S_g = state + (((size_t)slots[s] * H + h) * VS + (col ? j : 0)) * D + r * DR;
    float S[DR];
#pragma unroll
    for (int i = 0; i < DR; i += 4) {
        if constexpr (VEC) {
            const bool in = col && r * DR + i < D;      // (D % 4 == 0: a piece is inside or outside as a whole)
            const float4 x = in ? *(const float4*)(S_g + i) : make_float4(0.f, 0.f, 0.f, 0.f);
            S[i] = x.x; S[i + 1] = x.y; S[i + 2] = x.z; S[i + 3] = x.w;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) S[i + e] = (col && r * DR + i + e < D) ? S_g[i + e] : 0.f;
        }
    }
    const float keep_fixed = keep_const ? keep[h] : 0.f;
    float nxt[NL][W], v_nxt[P], a_nxt[P], b_nxt[P];
    auto fetch = [&](int first) {
#pragma unroll
        for (int n = 0; n < NL; ++n) {
            const int idx = n * NT + tid, p = idx / PIECES, e = (idx - p * PIECES) * W, which = e / DP, row = e - which * DP;
            const int t = first + p;
            const bool ok = idx < P * PIECES && t < t1 && row < D;
            const float* src = which == 0 ? k + (size_t)t * ldk + (size_t)g * D : q + (size_t)t * ldq + (size_t)g * D;
            if constexpr (VEC) {
                const float4 x = ok ? *(const float4*)(src + row) : make_float4(0.f, 0.f, 0.f, 0.f);
                nxt[n][0] = x.x; nxt[n][W - 3] = x.y; nxt[n][W - 2] = x.z; nxt[n][W - 1] = x.w;
            } else {
                nxt[n][0] = ok ? src[row] : 0.f;
            }
        }
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const bool live = first + p < t1;
            v_nxt[p] = (live && col) ? (ones ? 1.0f : v[(size_t)(first + p) * ldv + (size_t)h * V + j]) : 0.f;
            a_nxt[p] = live ? (keep_const ? keep_fixed : keep[(size_t)(first + p) * H + h]) : 1.f;
            b_nxt[p] = live ? (take ? take[(size_t)(first + p) * H + h] : 1.f) : 0.f;
        }
    };
    auto stage = [&](int slot) {
#pragma unroll
        for (int n = 0; n < NL; ++n) {
            const int idx = n * NT + tid;
            if (idx < P * PIECES) {
                float* dst = &kq[slot][0][0][0] + (size_t)idx * W;
                if constexpr (VEC) *(float4*)dst = make_float4(nxt[n][0], nxt[n][W - 3], nxt[n][W - 2], nxt[n][W - 1]);
                else *dst = nxt[n][0];
            }
        }
    };
    fetch(t0);
    stage(0);
    __syncthreads();
    for (int first = t0, cur = 0; first < t1; first += P, cur ^= 1) {
        float bv_cur[P], a_cur[P];
#pragma unroll
        for (int p = 0; p < P; ++p) {
            bv_cur[p] = b_nxt[p] * v_nxt[p];
            a_cur[p] = a_nxt[p];
        }
        const bool more = first + P < t1;
        if (more) fetch(first + P);                  // the next group's operands leave now and are staged after this group's work
        auto token = [&](int p, int t) {
            const float* kk = &kq[cur][p][0][r * DR];
            const float* qq = &kq[cur][p][1][r * DR];
            float sq = 0.f;
#pragma unroll
            for (int i = 0; i < DR; i += 4) {
                const float4 k4 = *(const float4*)(kk + i), q4 = *(const float4*)(qq + i);
                const float ka[4] = {k4.x, k4.y, k4.z, k4.w}, qa[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    S[i + e] = fmaf(ka[e], bv_cur[p], S[i + e] * a_cur[p]);
                    sq = fmaf(S[i + e], qa[e], sq);
                }
            }
            sq = column_sum<LPC>(sq) * q_scale;
            if (col && r == 0) {
                if (ones) nq[(size_t)t * H + h] = sq;
                else out[(size_t)t * ldo + (size_t)h * V + j] = sq;
            }
        };
        if (first + P <= t1) {
#pragma unroll
            for (int p = 0; p < P; ++p) token(p, first + p);
        } else {
#pragma unroll
            for (int p = 0; p < P; ++p)
                if (first + p < t1) token(p, first + p);
        }
        if (more) stage(cur ^ 1);                    // (the buffer that every wave left before the last barrier)
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < DR; i += 4) {
        if constexpr (VEC) {
            if (col && r * DR + i < D) *(float4*)(S_g + i) = make_float4(S[i], S[i + 1], S[i + 2], S[i + 3]);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (col && r * DR + i + e < D) S_g[i + e] = S[i + e];
        }
    }
}

FX_API int fx_gated_outer(void* stream, const float* q, long ldq, const float* k, long ldk, const float* v, long ldv,
                          const float* keep, int keep_const, const float* take, float* out, long ldo, float* nq, float* state,
                          const int* seq_starts, const int* slots, int n_seqs, int H, int G, int D, int V, float q_scale) {
    FX_REQUIRE(n_seqs >= 0 && H > 0 && G > 0 && H % G == 0, "gated_outer: bad sizes sequences=%d H=%d G=%d", n_seqs, H, G);
    FX_REQUIRE(D >= 1 && D <= 256 && V >= 1, "gated_outer: key size %d (up to 256) and value size %d", D, V);
    FX_REQUIRE(ldq >= (long)G * D && ldk >= (long)G * D && ldv >= (long)H * V && ldo >= (long)H * V, "gated_outer: rows too short for %d heads", H);
    FX_REQUIRE(n_seqs <= 65535 && H <= 65535, "gated_outer: %d sequences of %d heads are more than a launch takes", n_seqs, H);
    FX_REQUIRE(keep, "gated_outer: the forgetting factors are missing");
    if (n_seqs == 0) return 0;
    const int VS = V + (nq ? 1 : 0);
    const bool vec = D % 4 == 0 && ldq % 4 == 0 && ldk % 4 == 0 && (((uintptr_t)state | (uintptr_t)q | (uintptr_t)k) % 16) == 0;
    hipStream_t s = (hipStream_t)stream;
#define FX_OUTER(DR_, LPC_, NW_)                                                                                              \
    do {                                                                                                                      \
        const int per_block = NW_ * 64 / LPC_;                                                                                \
        const dim3 grid((VS + per_block - 1) / per_block, H, n_seqs);                                                         \
        if (vec) gated_outer_kernel<DR_, LPC_, true, NW_><<<grid, NW_ * 64, 0, s>>>(q, ldq, k, ldk, v, ldv, keep, keep_const, take, out, ldo, nq, state, seq_starts, slots, H, G, D, V, VS, q_scale); \
        else gated_outer_kernel<DR_, LPC_, false, NW_><<<grid, NW_ * 64, 0, s>>>(q, ldq, k, ldk, v, ldv, keep, keep_const, take, out, ldo, nq, state, seq_starts, slots, H, G, D, V, VS, q_scale);    \
    } while (0)
    if (D <= 64 && V <= 32) FX_OUTER(4, 16, 2);
    else if (D <= 64) FX_OUTER(4, 16, 4);
    else if (D <= 128) FX_OUTER(4, 32, 4);
    else FX_OUTER(8, 32, 8);
#undef FX_OUTER
    FX_CHECK_LAUNCH("gated_outer");
    return 0;
}

// ---------------------------------------------------------------------------
// Exponential gates kept in range by a running maximum, per head, over each sequence's tokens in order.  From the
// projections x_i, x_f [T, H] (float32 rows):
//   i = cap tanh(x_i / cap),  f = logsigmoid(cap tanh(x_f / cap))             two logarithms
//   m_t = max(f + m_(t-1), i);  keep_t = exp(f + m_(t-1) - m_t);  take_t = exp(i - m_t)
// m is carried in state[slot, h] (zero at a sequence's start).  Outputs keep, take, m: float32 [T, H].
// The running maximum is a scan: token t maps m to max(m + f_t, i_t), and two such maps in a row are one of the same
// form, (f_a + f_b, max(i_a + f_b, i_b)); a wave takes 64 tokens at a time, a lane each, and combines them in six
// rounds.  One wave per (sequence, head).
// ---------------------------------------------------------------------------
__device__ __forceinline__ float log_sigmoid_f(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

__global__ __launch_bounds__(64) void exp_gate_scan_kernel(const float* __restrict__ xi, long ldi, const float* __restrict__ xf, long ldf,
                                                           float cap, float* __restrict__ keep, float* __restrict__ take,
                                                           float* __restrict__ m_out, float* __restrict__ state,
                                                           const int* __restrict__ seq_starts, const int* __restrict__ slots, int H) {
    const int h = blockIdx.x, s = blockIdx.y, lane = threadIdx.x;
    const int t0 = seq_starts[s], t1 = seq_starts[s + 1];
    if (t1 <= t0) return;
    float* carried = state + (size_t)slots[s] * H + h;
    float m_prev = *carried;
    for (int base = t0; base < t1; base += 64) {
        const int t = base + lane;
        const bool live = t < t1;
        float gi = -INFINITY, gf = 0.f;
        if (live) {
            gi = cap * tanhf(xi[(size_t)t * ldi + h] / cap);
            gf = log_sigmoid_f(cap * tanhf(xf[(size_t)t * ldf + h] / cap));
        }
        float F = gf, I = gi;                       // the map of this lane's token; then of all tokens up to it
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const float Fp = __shfl_up(F, d), Ip = __shfl_up(I, d);
            if (lane >= d) {
                I = fmaxf(Ip + F, I);
                F = Fp + F;
            }
        }
        const float m_t = fmaxf(m_prev + F, I);
        float m_before = __shfl_up(m_t, 1);
        if (lane == 0) m_before = m_prev;
        if (live) {
            keep[(size_t)t * H + h] = expf(gf + m_before - m_t);
            take[(size_t)t * H + h] = expf(gi - m_t);
            m_out[(size_t)t * H + h] = m_t;
        }
        m_prev = __shfl(m_t, min(63, t1 - 1 - base));
    }
    if (lane == 0) *carried = m_prev;
}

FX_API int fx_exp_gate_scan(void* stream, const float* xi, long ldi, const float* xf, long ldf, float cap, float* keep,
                            float* take, float* m_out, float* state, const int* seq_starts, const int* slots, int n_seqs, int H) {
    FX_REQUIRE(n_seqs >= 0 && n_seqs <= 65535 && H > 0 && ldi >= H && ldf >= H, "exp_gate_scan: bad sizes sequences=%d H=%d", n_seqs, H);
    FX_REQUIRE(cap > 0.f, "exp_gate_scan: a cap of %g", (double)cap);
    if (n_seqs == 0) return 0;
    exp_gate_scan_kernel<<<dim3(H, n_seqs), 64, 0, (hipStream_t)stream>>>(xi, ldi, xf, ldf, cap, keep, take, m_out, state, seq_starts, slots, H);
    FX_CHECK_LAUNCH("exp_gate_scan");
    return 0;
}

// ---------------------------------------------------------------------------
// The real-gated linear recurrent unit.  Per channel c, with u the convolved input and r_l, i_l the logits of the
// recurrence gate and the input gate (float32 rows):
//   a = exp(-rate sigmoid(r_l) softplus(lam[c]));   x = sqrt(1 - a^2) sigmoid(i_l) u          (fx_rglru_gates; the logits
//                                                     come as the products of the channels' parts leave them, plus a bias)
//   S_t = a_t S_(t-1) + x_t;   y_t = S_t gelu_tanh(b_t)                                        (fx_rglru_scan)
// b the other branch's projection; S is carried in state[slot, c] (float32, zero at a sequence's start).
// The scan: a block owns 64 channels of one sequence, a lane each; its NW waves cut the sequence's tokens into NW
// stretches.  Every wave first folds its stretch from zero into one map S -> A S + B, the maps of the stretches before
// a wave's own give the state it starts from, and a second pass over the stretch makes the outputs from that state.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rglru_gates_kernel(const float* __restrict__ u, long ldu, const float* __restrict__ logits,
                                                          const float* __restrict__ bias, const void* __restrict__ lam, int lam_dtype,
                                                          float rate, float* __restrict__ a, float* __restrict__ x, int C, int cb, long n) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const long t = idx / C;
    const int c = (int)(idx - t * C), j = c / cb, e = c - j * cb;
    // the gates' logits lie part by part: [token][part][recurrence gate | input gate][channel of the part]
    const size_t at = ((size_t)t * (C / cb) + j) * 2 * cb + e, bat = (size_t)j * 2 * cb + e;
    const float rl = logits[at] + (bias ? bias[bat] : 0.f), il = logits[at + cb] + (bias ? bias[bat + cb] : 0.f);
    const float r = 1.0f / (1.0f + expf(-rl)), i = 1.0f / (1.0f + expf(-il));
    const float log_a = -rate * r * softplus_f(load_as_float(lam, lam_dtype, c));
    const float av = expf(log_a);
    a[idx] = av;
    // 1 - a^2 = -expm1(2 log a): the difference itself would lose its digits where a is close to one
    x[idx] = sqrtf(fmaxf(-expm1f(2.0f * log_a), 0.f)) * i * u[t * ldu + c];
}

FX_API int fx_rglru_gates(void* stream, const float* u, long ldu, const float* logits, const float* bias,
                          const void* lam, int lam_dtype, float rate, float* a, float* x, int T, int C, int n_parts) {
    FX_REQUIRE(T >= 0 && C > 0 && ldu >= C && n_parts >= 1 && C % n_parts == 0, "rglru_gates: bad sizes T=%d C=%d parts=%d", T, C, n_parts);
    FX_REQUIRE(lam_dtype == FX_F32 || lam_dtype == FX_BF16, "rglru_gates: unknown dtype %d", lam_dtype);
    if (T == 0) return 0;
    const long n = (long)T * C;
    rglru_gates_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(u, ldu, logits, bias, lam, lam_dtype, rate, a, x, C, C / n_parts, n);
    FX_CHECK_LAUNCH("rglru_gates");
    return 0;
}

__device__ __forceinline__ float gelu_tanh_f(float z) { return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }

template <typename T, int NW>
__global__ __launch_bounds__(NW * 64) void rglru_scan_kernel(const float* __restrict__ a, const float* __restrict__ x,
                                                             const float* __restrict__ b, long ldb, T* __restrict__ y, long ldy,
                                                             float* __restrict__ state, const int* __restrict__ seq_starts,
                                                             const int* __restrict__ slots, int C) {
    __shared__ float A_of[NW][64], B_of[NW][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + lane, s = blockIdx.y;
    const int t0 = seq_starts[s], t1 = seq_starts[s + 1];
    if (t1 <= t0) return;                            // (the same in every thread of the block)
    const int n = t1 - t0, per = (n + NW - 1) / NW;
    const int w0 = min(t0 + wave * per, t1), w1 = min(w0 + per, t1);
    const bool in = c < C;
    constexpr int P = 8;                             // tokens whose operands are asked for together
    float A = 1.f, B = 0.f;
    if (NW > 1) {
        if (in)
            for (int t = w0; t < w1; t += P) {
                float av[P], xv[P];
#pragma unroll
                for (int p = 0; p < P; ++p) {            // (past the stretch: the map that changes nothing)
                    const bool live = t + p < w1;
                    av[p] = live ? a[(size_t)(t + p) * C + c] : 1.f;
                    xv[p] = live ? x[(size_t)(t + p) * C + c] : 0.f;
                }
#pragma unroll
                for (int p = 0; p < P; ++p) {
                    B = fmaf(av[p], B, xv[p]);
                    A *= av[p];
                }
            }
        A_of[wave][lane] = A;
        B_of[wave][lane] = B;
        __syncthreads();
    }
    float S = in ? state[(size_t)slots[s] * C + c] : 0.f;
    for (int w = 0; w < wave; ++w) S = fmaf(A_of[w][lane], S, B_of[w][lane]);
    if (!in) return;
    for (int t = w0; t < w1; t += P) {
        float av[P], xv[P], bv[P];
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const bool live = t + p < w1;
            av[p] = live ? a[(size_t)(t + p) * C + c] : 1.f;
            xv[p] = live ? x[(size_t)(t + p) * C + c] : 0.f;
            bv[p] = live ? b[(size_t)(t + p) * ldb + c] : 0.f;
        }
#pragma unroll
        for (int p = 0; p < P; ++p) {
            S = fmaf(av[p], S, xv[p]);
            if (t + p < w1) from_float(y + (size_t)(t + p) * ldy + c, S * gelu_tanh_f(bv[p]));
        }
    }
    if (wave == NW - 1) state[(size_t)slots[s] * C + c] = S;
}

FX_API int fx_rglru_scan(void* stream, int out_dtype, const float* a, const float* x, const float* b, long ldb, void* y, long ldy,
                         float* state, const int* seq_starts, const int* slots, int n_seqs, int C, int longest) {
    FX_REQUIRE(n_seqs >= 0 && n_seqs <= 65535 && C > 0 && ldb >= C && ldy >= C, "rglru_scan: bad sizes sequences=%d C=%d", n_seqs, C);
    FX_REQUIRE(out_dtype == FX_F32 || out_dtype == FX_BF16, "rglru_scan: unknown output dtype %d", out_dtype);
    if (n_seqs == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((C + 63) / 64, n_seqs);
#define FX_SCAN(T_, NW_) rglru_scan_kernel<T_, NW_><<<grid, NW_ * 64, 0, s>>>(a, x, b, ldb, (T_*)y, ldy, state, seq_starts, slots, C)
    // (`longest`: the most tokens any sequence brings; it picks how many waves cut a sequence, nothing else)
    if (out_dtype == FX_F32) {
        if (longest <= 16) FX_SCAN(float, 1);
        else if (longest <= 256) FX_SCAN(float, 4);
        else FX_SCAN(float, 16);
    } else {
        if (longest <= 16) FX_SCAN(bf16, 1);
        else if (longest <= 256) FX_SCAN(bf16, 4);
        else FX_SCAN(bf16, 16);
    }
#undef FX_SCAN
    FX_CHECK_LAUNCH("rglru_scan");
    return 0;
}
