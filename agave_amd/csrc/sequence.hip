// Kernels of the mixers that carry a state from token to token, and of the attention whose
// heads talk to each other, for gfx950:
//
//   short causal convolution per channel, with the last taps - 1 inputs of a sequence as state;
//   per-head RMS norm + rotation (pairs interleaved or split in halves) + cache write, for key and
//     value heads of different sizes, pages stored row by row;
//   attention over the paged cache with the heads' scores mixed by a matrix before the softmax,
//     keys of the query's own chunk only (or all earlier keys), a gate per head;
//   the gated linear recurrence S <- diag(a) S + k u^T, o = S^T q with u = beta (v - S^T k) (delta
//     rule) or u = v (forget-gate form), the gates made inside by waves of their own;
//   per-head RMS norm of the read-out with an optional elementwise sigmoid gate.
//
// Everything between the first product of a mixer and the rows its output product reads is 32-bit
// here: projections arrive as float rows, state is float, angles are made in double.  T is the
// element type of the cache pages and of the rows handed to the output product.
#include "common_impl.h"
#include <math.h>

#define CONV_MAX_TAPS 8

// Gates by the hardware's exponential, logarithm and reciprocal (an ulp or two each, absolute errors of
// about 1e-7 in a gate that lies in (0, 1)): the library's exact versions are 15 to 30 instructions each, and
// the recurrence's producer waves, which share their SIMDs with the waves that run the chain, spent most of
// theirs on them.
__device__ __forceinline__ float sigmoid_f(float x) { return __frcp_rn(1.0f + __expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x * sigmoid_f(x); }
__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : __logf(1.0f + __expf(x)); }
__device__ __forceinline__ float decay_f(float rate, float x) { return __expf(-rate * softplus_f(x)); }

// ------------------------------------------------------------------ short causal convolution
//   y[t][c] = act(bias[c] + sum_j w[c][j] * u[pos(t) - taps + 1 + j][c]),  zeros before the sequence's start
//   (bias may be null).
// Inputs older than the step's first token come from state[slot][taps - 1][C], which holds the
// inputs at positions pos0 - taps + 1 .. pos0 - 1.  fused_update (every sequence brings one token):
// the thread that owns (sequence, channel) also shifts the state; otherwise conv_state_kernel does
// it afterwards, when no thread reads the old state any more.
template <bool SILU>
__global__ void short_conv_kernel(const float* __restrict__ u, long ldu, const float* __restrict__ w,
                                  const float* __restrict__ bias, float* __restrict__ y, long ldy, float* __restrict__ state,
                                  const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                  const int* __restrict__ pos0, const int* __restrict__ slots, int C, int taps,
                                  int fused_update, const float* __restrict__ in_bias) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int t = blockIdx.y;
    if (c >= C) return;
    const int s = tok_seq[t], p = tok_pos[t], p0 = pos0[s];
    float* st_c = state + ((size_t)slots[s] * (taps - 1)) * C + c;
    const float ib = in_bias ? in_bias[c] : 0.f;            // added to every input of the step (the state holds inputs with it)
    float in[CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
        in[j] = 0.f;
        if (j < taps) {
            const int r = p - taps + 1 + j;                 // position of this tap's input
            if (r >= p0) in[j] = u[(size_t)(t - (p - r)) * ldu + c] + ib;
            else in[j] = st_c[(size_t)(r - (p0 - (taps - 1))) * C];
        }
    }
    float acc = bias ? bias[c] : 0.f;
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j)
        if (j < taps) acc = fmaf(w[(size_t)c * taps + j], in[j], acc);
    y[(size_t)t * ldy + c] = SILU ? silu_f(acc) : acc;
    if (fused_update) {
#pragma unroll
        for (int j = 1; j < CONV_MAX_TAPS; ++j)
            if (j < taps) st_c[(size_t)(j - 1) * C] = in[j];
    }
}

__global__ void conv_state_kernel(const float* __restrict__ u, long ldu, float* __restrict__ state,
                                  const int* __restrict__ cu, const int* __restrict__ pos0,
                                  const int* __restrict__ slots, int C, int taps, const float* __restrict__ in_bias) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int s = blockIdx.y;
    if (c >= C) return;
    const int r0 = cu[s], n = cu[s + 1] - r0;
    float* st_c = state + ((size_t)slots[s] * (taps - 1)) * C + c;
    float keep[CONV_MAX_TAPS];
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS - 1; ++i) {
        keep[i] = 0.f;
        if (i < taps - 1) {
            const int back = taps - 1 - i;                  // the input `back` positions before the new end
            if (back <= n) keep[i] = u[(size_t)(r0 + n - back) * ldu + c] + (in_bias ? in_bias[c] : 0.f);
            else keep[i] = st_c[(size_t)(i + n) * C];
        }
    }
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS - 1; ++i)
        if (i < taps - 1) st_c[(size_t)i * C] = keep[i];
}

extern "C" int agave_short_conv(const float* u, long ldu, const float* w, const float* bias, float* y, long ldy, float* state,
                                const int* tok_seq, const int* tok_pos, const int* cu, const int* pos0,
                                const int* slots, int n_tokens, int n_seqs, int C, int taps, int silu,
                                int one_token_each, const float* in_bias, hipStream_t stream) {
    AGAVE_CHECK(n_tokens >= 0 && n_seqs >= 0 && C > 0, "short_conv: bad sizes N=%d B=%d C=%d", n_tokens, n_seqs, C);
    AGAVE_CHECK(taps >= 1 && taps <= CONV_MAX_TAPS, "short_conv: %d taps (1 to %d are supported)", taps, CONV_MAX_TAPS);
    AGAVE_CHECK(ldu >= C && ldy >= C, "short_conv: a row stride is below %d", C);
    AGAVE_CHECK(u && w && y && (state || taps == 1) && tok_seq && tok_pos && cu && pos0 && slots, "short_conv: null buffer");
    AGAVE_CHECK(u != y, "short_conv: the convolution is not done in place");
    AGAVE_CHECK(n_tokens < 65536 * 16, "short_conv: too many tokens");
    if (n_tokens == 0) return 0;
    const int threads = C >= 256 ? 256 : 64;
    const dim3 grid((C + threads - 1) / threads, n_tokens);
    if (silu)
        short_conv_kernel<true><<<grid, threads, 0, stream>>>(u, ldu, w, bias, y, ldy, state, tok_seq, tok_pos, pos0, slots, C, taps, one_token_each, in_bias);
    else
        short_conv_kernel<false><<<grid, threads, 0, stream>>>(u, ldu, w, bias, y, ldy, state, tok_seq, tok_pos, pos0, slots, C, taps, one_token_each, in_bias);
    AGAVE_LAUNCH_CHECK("short_conv");
    if (!one_token_each && taps > 1) {
        conv_state_kernel<<<dim3((C + threads - 1) / threads, n_seqs), threads, 0, stream>>>(u, ldu, state, cu, pos0, slots, C, taps, in_bias);
        AGAVE_LAUNCH_CHECK("conv_state");
    }
    return 0;
}

// ------------------------------------------------------------------ head norm + rotation + cache rows
// A wave per (token, head).  Heads 0 .. nh-1 are queries (written to q_out as float rows), the next
// nkv are keys (into k_pages [page][kv head][64][dk]) and the last nkv values (copied into v_pages
// [page][kv head][64][dv]).  Norm: x * rsqrt(mean(x^2) + eps) * gain (gain may be null).  Rotation of
// the first 2 * rot_half elements: interleaved pairs (2i, 2i+1) or halves (i, i + rot_half); the pair
// (a, b) at position p becomes (a cos - b sin, b cos + a sin), angle p * freq[i] made in double.
template <typename T>
__global__ __launch_bounds__(64) void head_norm_rope_rows_kernel(
    const float* __restrict__ q, long ldq, const float* __restrict__ k, long ldk, const float* __restrict__ v, long ldv,
    float* __restrict__ q_out, long ldqo, const float* __restrict__ q_gain, const float* __restrict__ k_gain,
    float eps_q, float eps_k, int norm_q, int norm_k, const double* __restrict__ freq, int rot_half, int interleaved,
    const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, T* __restrict__ k_pages, T* __restrict__ v_pages,
    const int* __restrict__ table, int width, const int* __restrict__ base, int n_pages, int nh, int nkv, int dk, int dv) {
    const int per_tok = nh + 2 * nkv;
    const int t = blockIdx.x / per_tok, head = blockIdx.x % per_tok;
    const int lane = threadIdx.x;
    const int p = tok_pos[t];
    long row = -1;                                          // row of the cache this head is written to
    if (head >= nh) {
        const int b = tok_seq[t];
        const int col = p / AGAVE_PAGE - base[b];
        int pg = (col >= 0 && col < width) ? table[(size_t)b * width + col] : -1;
        if (pg < 0 || pg >= n_pages) return;               // the planner never leaves such a hole
        const int kvh = head >= nh + nkv ? head - nh - nkv : head - nh;
        row = ((long)pg * nkv + kvh) * AGAVE_PAGE + (p % AGAVE_PAGE);
    }
    if (head >= nh + nkv) {
        const float* x = v + (size_t)t * ldv + (size_t)(head - nh - nkv) * dv;
        T* o = v_pages + (size_t)row * dv;
        for (int d = lane; d < dv; d += 64) st(o + d, x[d]);
        return;
    }
    const bool is_q = head < nh;
    const float* x = is_q ? q + (size_t)t * ldq + (size_t)head * dk : k + (size_t)t * ldk + (size_t)(head - nh) * dk;
    const float* gain = is_q ? q_gain : k_gain;
    const bool normed = is_q ? norm_q : norm_k;
    float inv = 1.f;
    if (normed) {
        float ss = 0.f;
        for (int d = lane; d < dk; d += 64) ss = fmaf(x[d], x[d], ss);
        ss = wave_sum(ss);
        inv = 1.0f / sqrtf(ss / (float)dk + (is_q ? eps_q : eps_k));
    }
    for (int d = lane; d < dk; d += 64) {
        float val = x[d] * inv * (gain ? gain[d] : 1.f);
        if (d < 2 * rot_half) {
            int fi, other;
            bool first;
            if (interleaved) { fi = d >> 1; other = d ^ 1; first = !(d & 1); }
            else { fi = d < rot_half ? d : d - rot_half; other = d < rot_half ? d + rot_half : d - rot_half; first = d < rot_half; }
            const float oth = x[other] * inv * (gain ? gain[other] : 1.f);
            const double ang = (double)p * freq[fi];
            const float c = (float)cos(ang), s = (float)sin(ang);
            val = first ? val * c - oth * s : val * c + oth * s;
        }
        if (is_q) q_out[(size_t)t * ldqo + (size_t)head * dk + d] = val;
        else st(k_pages + (size_t)row * dk + d, val);
    }
}

extern "C" int agave_head_norm_rope_rows(int dtype, const float* q, long ldq, const float* k, long ldk, const float* v,
                                         long ldv, float* q_out, long ldqo, const float* q_gain, const float* k_gain,
                                         float eps_q, float eps_k, int norm_q, int norm_k, const double* freq,
                                         int rot_half, int interleaved, const int* tok_seq, const int* tok_pos,
                                         void* k_pages, void* v_pages, const int* table, int width, const int* base,
                                         int n_pages, int N, int nh, int nkv, int dk, int dv, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && nh >= 0 && nkv >= 0 && dk > 0 && dv > 0, "head_norm_rope_rows: bad sizes N=%d nh=%d nkv=%d dk=%d dv=%d", N, nh, nkv, dk, dv);
    AGAVE_CHECK(rot_half >= 0 && 2 * rot_half <= dk, "head_norm_rope_rows: %d rotated elements exceed the head's %d", 2 * rot_half, dk);
    AGAVE_CHECK(rot_half == 0 || freq, "head_norm_rope_rows: rotation without a frequency table");
    AGAVE_CHECK(nh == 0 || (q && q_out && ldq >= (long)nh * dk && ldqo >= (long)nh * dk), "head_norm_rope_rows: bad q buffers");
    AGAVE_CHECK(nkv == 0 || (k && v && k_pages && v_pages && table && base && width > 0 && n_pages > 0 &&
                             ldk >= (long)nkv * dk && ldv >= (long)nkv * dv), "head_norm_rope_rows: bad k/v buffers");
    AGAVE_CHECK(tok_seq && tok_pos, "head_norm_rope_rows: null token tables");
    AGAVE_CHECK((long)N * (nh + 2 * nkv) < 2147483647L, "head_norm_rope_rows: too many rows");
    if (N == 0 || nh + nkv == 0) return 0;
    const int grid = N * (nh + 2 * nkv);
    if (dtype == AGAVE_F32)
        head_norm_rope_rows_kernel<float><<<grid, 64, 0, stream>>>(q, ldq, k, ldk, v, ldv, q_out, ldqo, q_gain, k_gain, eps_q, eps_k,
            norm_q, norm_k, freq, rot_half, interleaved, tok_seq, tok_pos, (float*)k_pages, (float*)v_pages, table, width, base,
            n_pages, nh, nkv, dk, dv);
    else if (dtype == AGAVE_BF16)
        head_norm_rope_rows_kernel<bf16><<<grid, 64, 0, stream>>>(q, ldq, k, ldk, v, ldv, q_out, ldqo, q_gain, k_gain, eps_q, eps_k,
            norm_q, norm_k, freq, rot_half, interleaved, tok_seq, tok_pos, (bf16*)k_pages, (bf16*)v_pages, table, width, base,
            n_pages, nh, nkv, dk, dv);
    else
        AGAVE_CHECK(false, "head_norm_rope_rows: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("head_norm_rope_rows");
    return 0;
}

// ------------------------------------------------------------------ attention with talking heads
// A workgroup per query token, all heads at once (the mixing needs every head's score of a key):
//   raw[g][j]  = scale * q_g . k_j            (key head of g: g / (nh / nkv))
//   s[h][j]    = sum_g talk[h][g] raw[g][j]   (talk null: s = raw)
//   w[h][.]    = softmax over the visible keys j: j <= p, and j >= floor(p / chunk) * chunk if chunk > 0
//   out[h]     = sigmoid(gate[h]) * out_scale * sum_j w[h][j] v_j
// Keys come in tiles of 64 with a running maximum and sum per head.  Dynamic LDS:
//   qs[nh*dk] raw[nh*64] mix[nh*64] talk[nh*nh] m[nh] l[nh] alpha[nh] pg[64] vt[64*vcols]
#define TALK_ACC_MAX 16          // sums a thread: heads x value size up to 256 times this
template <typename T, int TALK_ACC>
__global__ __launch_bounds__(256) void talk_attention_kernel(
    const float* __restrict__ q, long ldq, const float* __restrict__ gate, long ldg, T* __restrict__ out, long ldo,
    const T* __restrict__ k_pages, const T* __restrict__ v_pages, const int* __restrict__ table, int width,
    const int* __restrict__ base, int n_pages, const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
    const float* __restrict__ talk, int nh, int nkv, int dk, int dv, float scale, int chunk, float out_scale, int vcols,
    float* __restrict__ parts, int tiles) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    float* qs = lds;
    float* raw = qs + (size_t)nh * dk;
    float* mix = raw + (size_t)nh * 64;
    float* tk = mix + (size_t)nh * 64;
    float* m_run = tk + (size_t)nh * nh;
    float* l_run = m_run + nh;
    float* alpha = l_run + nh;
    int* pg = reinterpret_cast<int*>(alpha + nh);
    // [64 keys][vcols], on a 16-byte boundary
    float* vt = lds + (((size_t)nh * dk + 2 * (size_t)nh * 64 + (size_t)nh * nh + 3 * (size_t)nh + 64 + 3) & ~(size_t)3);

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int t = blockIdx.x;
    const int b = tok_seq[t], p = tok_pos[t];
    const int lo = chunk > 0 ? (p / chunk) * chunk : 0;
    const int rep = nh / nkv;
    const int pbase = base[b];

    for (int i = tid; i < nh * dk; i += 256) qs[i] = q[(size_t)t * ldq + i];
    if (talk)
        for (int i = tid; i < nh * nh; i += 256) tk[i] = talk[i];
    for (int i = tid; i < nh; i += 256) { m_run[i] = -INFINITY; l_run[i] = 0.f; }
    float acc[TALK_ACC];
#pragma unroll
    for (int a = 0; a < TALK_ACC; ++a) acc[a] = 0.f;
    // which outputs a thread sums: elements tid + 256 a of the token's [nh][dv] row (head and element kept:
    // no division inside the loops)
    int one_h[TALK_ACC];                                    // head of accumulator a (nh: none)
#pragma unroll
    for (int a = 0; a < TALK_ACC; ++a) {
        const int idx = tid + a * 256;
        one_h[a] = idx < nh * dv ? idx / dv : nh;
    }
    __syncthreads();

    // parts: the launch has a workgroup per tile of 64 keys (blockIdx.y) and key head (blockIdx.z), which leaves
    // its heads' sums, maximum and weight for talk_merge_kernel; a tile behind the query's position leaves none (weight 0)
    const int j_first = parts ? lo + (int)blockIdx.y * 64 : lo;
    const int j_last = parts ? (j_first + 63 < p ? j_first + 63 : p) : p;
    for (int j0 = j_first; j0 <= j_last; j0 += 64) {
        const int nk = p - j0 + 1 < 64 ? p - j0 + 1 : 64;
        if (tid < 64) {
            int id = -1;
            const int j = j0 + tid;
            if (tid < nk) {
                const int col = j / AGAVE_PAGE - pbase;
                if (col >= 0 && col < width) id = table[(size_t)b * width + col];
                if (id >= n_pages) id = -1;
            }
            pg[tid] = id;
        }
        __syncthreads();
        // raw scores: lane = key; a wave takes up to four query heads of one key head at a time, so a
        // key row is read once for them (16 bytes a load where the row's size allows)
        {
            const int j = j0 + lane;
            const int id = pg[lane];
            const int quads = (rep + 3) / 4, items = nkv * quads;
            for (int it = wv; it < items; it += 4) {
                const int g = it / quads, h0 = g * rep + (it % quads) * 4;
                const int nq = g * rep + rep - h0 < 4 ? g * rep + rep - h0 : 4;
                const float* q0 = qs + (size_t)h0 * dk;
                const float* q1 = qs + (size_t)(h0 + (nq > 1 ? 1 : 0)) * dk;
                const float* q2 = qs + (size_t)(h0 + (nq > 2 ? 2 : 0)) * dk;
                const float* q3 = qs + (size_t)(h0 + (nq > 3 ? 3 : 0)) * dk;
                float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
                if (id >= 0) {
                    const T* kr = k_pages + (((size_t)id * nkv + g) * AGAVE_PAGE + (j % AGAVE_PAGE)) * dk;
                    constexpr int VE = 16 / sizeof(T);                  // elements of a 16-byte load
                    if (dk % VE == 0) {
                        auto use = [&](const uint4& raw16, int d) {
                            float kf[VE];
                            if (sizeof(T) == 2) {
                                const uint32_t w[4] = {raw16.x, raw16.y, raw16.z, raw16.w};
#pragma unroll
                                for (int i = 0; i < 4; ++i) {
                                    kf[(2 * i) % VE] = __builtin_bit_cast(float, w[i] << 16);
                                    kf[(2 * i + 1) % VE] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
                                }
                            } else {
                                kf[0] = __builtin_bit_cast(float, raw16.x); kf[1] = __builtin_bit_cast(float, raw16.y);
                                kf[2] = __builtin_bit_cast(float, raw16.z); kf[3] = __builtin_bit_cast(float, raw16.w);
                            }
#pragma unroll
                            for (int i = 0; i < VE; i += 4) {           // dk is a multiple of 4 here: whole float4s of q
                                const float4 a0 = *reinterpret_cast<const float4*>(q0 + d + i);
                                const float4 a1 = *reinterpret_cast<const float4*>(q1 + d + i);
                                const float4 a2 = *reinterpret_cast<const float4*>(q2 + d + i);
                                const float4 a3 = *reinterpret_cast<const float4*>(q3 + d + i);
                                d0 = fmaf(a0.x, kf[i], d0); d0 = fmaf(a0.y, kf[i + 1], d0); d0 = fmaf(a0.z, kf[i + 2], d0); d0 = fmaf(a0.w, kf[i + 3], d0);
                                d1 = fmaf(a1.x, kf[i], d1); d1 = fmaf(a1.y, kf[i + 1], d1); d1 = fmaf(a1.z, kf[i + 2], d1); d1 = fmaf(a1.w, kf[i + 3], d1);
                                d2 = fmaf(a2.x, kf[i], d2); d2 = fmaf(a2.y, kf[i + 1], d2); d2 = fmaf(a2.z, kf[i + 2], d2); d2 = fmaf(a2.w, kf[i + 3], d2);
                                d3 = fmaf(a3.x, kf[i], d3); d3 = fmaf(a3.y, kf[i + 1], d3); d3 = fmaf(a3.z, kf[i + 2], d3); d3 = fmaf(a3.w, kf[i + 3], d3);
                            }
                        };
                        const uint4* k16 = reinterpret_cast<const uint4*>(kr);
                        const int n16 = dk / VE;
                        int c = 0;
                        for (; c + 4 <= n16; c += 4) {                  // four loads on their way before the first is used
                            uint4 b[4];
#pragma unroll
                            for (int i = 0; i < 4; ++i) b[i] = k16[c + i];
#pragma unroll
                            for (int i = 0; i < 4; ++i) use(b[i], (c + i) * VE);
                        }
                        for (; c < n16; ++c) use(k16[c], c * VE);
                    } else {
                        for (int d = 0; d < dk; ++d) {
                            const float kv = ld(kr + d);
                            d0 = fmaf(q0[d], kv, d0); d1 = fmaf(q1[d], kv, d1);
                            d2 = fmaf(q2[d], kv, d2); d3 = fmaf(q3[d], kv, d3);
                        }
                    }
                }
                raw[h0 * 64 + lane] = d0 * scale;
                if (nq > 1) raw[(h0 + 1) * 64 + lane] = d1 * scale;
                if (nq > 2) raw[(h0 + 2) * 64 + lane] = d2 * scale;
                if (nq > 3) raw[(h0 + 3) * 64 + lane] = d3 * scale;
            }
        }
        __syncthreads();
        // mixing, then each head's running maximum and sum (a wave per head in turn)
        for (int h = wv; h < nh; h += 4) {
            float s;
            if (talk) {
                s = 0.f;
                for (int g = 0; g < nh; ++g) s = fmaf(tk[h * nh + g], raw[g * 64 + lane], s);
            } else {
                s = raw[h * 64 + lane];
            }
            const bool valid = lane < nk && pg[lane] >= 0;
            if (!valid) s = -INFINITY;
            const float tmax = wave_max(s);
            const float m_old = m_run[h];
            const float m_new = fmaxf(m_old, tmax);
            const float al = (m_old == -INFINITY) ? 0.f : expf(m_old - m_new);
            const float pr = valid ? expf(s - m_new) : 0.f;
            mix[h * 64 + lane] = pr;
            const float sum = wave_sum(pr);
            if (lane == 0) {
                m_run[h] = m_new;
                l_run[h] = l_run[h] * al + sum;
                alpha[h] = al;
            }
        }
        __syncthreads();
        // weighted sum of the values: a thread per (head, value element); the tile's values of one key
        // head (up to vcols columns at a time) come into LDS once, in whole rows, and every head of
        // the group reads them there
#pragma unroll
        for (int a = 0; a < TALK_ACC; ++a) {
            if (one_h[a] < nh) acc[a] *= alpha[one_h[a]];
        }
        // (with parts, a workgroup sums the values of one key head only: blockIdx.z; the scores it needs all)
        const int g_first = parts ? (int)blockIdx.z : 0, g_end = parts ? g_first + 1 : nkv;
        for (int g = g_first; g < g_end; ++g) {
            for (int e0 = 0; e0 < dv; e0 += vcols) {
                const int ec = dv - e0 < vcols ? dv - e0 : vcols;
                __syncthreads();                                   // the tile before is read
                // a wave takes the rows wv, wv + 4, ...; four rows' loads leave before the first is stored
                // (from clamped addresses, so that none stands under a condition)
                if (pg[0] >= 0) {
                    for (int u0 = 0; u0 < 16; u0 += 4) {
                        if (wv + 4 * u0 >= nk) break;
                        const T* rowp[4];
                        bool ok[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int r = wv + 4 * (u0 + u);
                            ok[u] = r < nk && pg[r] >= 0;
                            const int rr = ok[u] ? r : 0;
                            rowp[u] = v_pages + (((size_t)pg[rr] * nkv + g) * AGAVE_PAGE + ((j0 + rr) % AGAVE_PAGE)) * dv + e0;
                        }
                        for (int c0 = 0; c0 < ec; c0 += 64) {
                            const int e = c0 + lane, ee = e < ec ? e : 0;
                            T got[4];
#pragma unroll
                            for (int u = 0; u < 4; ++u) got[u] = rowp[u][ee];
#pragma unroll
                            for (int u = 0; u < 4; ++u) {
                                const int r = wv + 4 * (u0 + u);
                                if (r < nk && e < ec) vt[r * vcols + e] = ok[u] ? ld(&got[u]) : 0.f;
                            }
                        }
                    }
                }
                __syncthreads();
                {
#pragma unroll
                    for (int a = 0; a < TALK_ACC; ++a) {
                        const int e = tid + a * 256 - one_h[a] * dv - e0;
                        if (one_h[a] >= g * rep && one_h[a] < (g + 1) * rep && e >= 0 && e < ec) {
                            const float* w = mix + one_h[a] * 64;
                            const float* x = vt + e;
                            float s0 = 0.f, s1 = 0.f;
                            int r = 0;
                            for (; r + 1 < nk; r += 2) {
                                s0 = fmaf(w[r], x[r * vcols], s0);
                                s1 = fmaf(w[r + 1], x[(r + 1) * vcols], s1);
                            }
                            if (r < nk) s0 = fmaf(w[r], x[r * vcols], s0);
                            acc[a] += s0 + s1;
                        }
                    }
                }
            }
        }
        __syncthreads();
    }
    if (parts) {
        float* mine = parts + ((size_t)t * tiles + blockIdx.y) * nh * (dv + 2);
#pragma unroll
        for (int a = 0; a < TALK_ACC; ++a) {
            const int h = one_h[a];
            if (h < nh && h / rep == (int)blockIdx.z) mine[(size_t)h * (dv + 2) + (tid + a * 256 - h * dv)] = acc[a];
        }
        for (int h = tid; h < nh; h += 256) {
            if (h / rep != (int)blockIdx.z) continue;
            mine[(size_t)h * (dv + 2) + dv] = m_run[h];
            mine[(size_t)h * (dv + 2) + dv + 1] = l_run[h];
        }
        return;
    }
#pragma unroll
    for (int a = 0; a < TALK_ACC; ++a) {
        const int h = one_h[a], idx = tid + a * 256;
        if (h < nh) {
            const float l = l_run[h];
            float o = l > 0.f ? acc[a] / l : 0.f;
            if (gate) o *= sigmoid_f(gate[(size_t)t * ldg + h]);
            st(out + (size_t)t * ldo + idx, o * out_scale);
        }
    }
}

// The tiles' partial results of one (token, head) put together: a wave per pair.
template <typename T>
__global__ __launch_bounds__(64) void talk_merge_kernel(const float* __restrict__ parts, int tiles, const float* __restrict__ gate,
                                                        long ldg, T* __restrict__ out, long ldo, int nh, int dv, float out_scale) {
    const int t = blockIdx.x / nh, h = blockIdx.x % nh, lane = threadIdx.x;
    const float* mine = parts + ((size_t)t * tiles * nh + h) * (dv + 2);
    const size_t step = (size_t)nh * (dv + 2);
    float m = -INFINITY;
    for (int i = 0; i < tiles; ++i)
        if (mine[i * step + dv + 1] > 0.f) m = fmaxf(m, mine[i * step + dv]);
    float l = 0.f;
    for (int i = 0; i < tiles; ++i)
        if (mine[i * step + dv + 1] > 0.f) l += expf(mine[i * step + dv] - m) * mine[i * step + dv + 1];
    const float g = (gate ? sigmoid_f(gate[(size_t)t * ldg + h]) : 1.f) * out_scale / (l > 0.f ? l : 1.f);
    for (int e = lane; e < dv; e += 64) {
        float sum = 0.f;
        for (int i = 0; i < tiles; ++i)
            if (mine[i * step + dv + 1] > 0.f) sum = fmaf(expf(mine[i * step + dv] - m), mine[i * step + e], sum);
        st(out + (size_t)t * ldo + (size_t)h * dv + e, sum * g);
    }
}

extern "C" int agave_talk_attention(int dtype, const float* q, long ldq, const float* gate, long ldg, void* out, long ldo,
                                    const void* k_pages, const void* v_pages, const int* table, int width,
                                    const int* base, int n_pages, const int* tok_seq, const int* tok_pos,
                                    const float* talk, int N, int nh, int nkv, int dk, int dv, float scale, int chunk,
                                    float out_scale, float* parts, int tiles, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && nh > 0 && nkv > 0 && dk > 0 && dv > 0, "talk_attention: bad sizes N=%d nh=%d nkv=%d dk=%d dv=%d", N, nh, nkv, dk, dv);
    AGAVE_CHECK(nh % nkv == 0, "talk_attention: %d query heads are not a multiple of %d key heads", nh, nkv);
    AGAVE_CHECK((long)nh * dv <= 256 * TALK_ACC_MAX, "talk_attention: heads x value size %ld exceeds %d", (long)nh * dv, 256 * TALK_ACC_MAX);
    AGAVE_CHECK(ldq >= (long)nh * dk && ldo >= (long)nh * dv && (!gate || ldg >= nh), "talk_attention: a row stride is too small");
    AGAVE_CHECK(chunk >= 0, "talk_attention: negative chunk");
    AGAVE_CHECK(q && out && k_pages && v_pages && table && base && tok_seq && tok_pos && width > 0 && n_pages > 0,
                "talk_attention: null buffer or empty table");
    const size_t fixed = ((size_t)nh * dk + 2 * (size_t)nh * 64 + (size_t)nh * nh + 3 * (size_t)nh + 64 + 4) * sizeof(float);
    int vcols = 128;                                        // value columns of a key head that are in LDS at a time
    while (vcols > 16 && (vcols / 2 >= dv || fixed + 64 * vcols * sizeof(float) > 64 * 1024)) vcols /= 2;
    const size_t lds = fixed + 64 * vcols * sizeof(float);
    AGAVE_CHECK(lds <= 64 * 1024, "talk_attention: %d heads of size %d need %zu bytes of LDS (64 KB are there)", nh, dk, lds);
    if (N == 0) return 0;
#define TALK_LAUNCH(T, ACC)                                                                                            \
    talk_attention_kernel<T, ACC><<<grid, 256, lds, stream>>>(q, ldq, gate, ldg, (T*)out, ldo, (const T*)k_pages,      \
        (const T*)v_pages, table, width, base, n_pages, tok_seq, tok_pos, talk, nh, nkv, dk, dv, scale, chunk, out_scale,  \
        vcols, parts, tiles)
    AGAVE_CHECK(!parts || (tiles >= 1 && tiles <= 1024 && chunk > 0 && (long)tiles * 64 >= chunk),
                "talk_attention: %d tiles of 64 keys do not cover a chunk of %d", tiles, chunk);
    const dim3 grid(N, parts ? tiles : 1, parts ? nkv : 1);
    const int sums = (nh * dv + 255) / 256;                 // a thread's sums: fewer registers where fewer do
    if (dtype == AGAVE_F32) {
        if (sums <= 4) TALK_LAUNCH(float, 4); else if (sums <= 8) TALK_LAUNCH(float, 8); else TALK_LAUNCH(float, 16);
    } else if (dtype == AGAVE_BF16) {
        if (sums <= 4) TALK_LAUNCH(bf16, 4); else if (sums <= 8) TALK_LAUNCH(bf16, 8); else TALK_LAUNCH(bf16, 16);
    } else {
        AGAVE_CHECK(false, "talk_attention: unknown dtype %d", dtype);
    }
#undef TALK_LAUNCH
    if (parts) {
        AGAVE_LAUNCH_CHECK("talk_attention");
        if (dtype == AGAVE_F32)
            talk_merge_kernel<float><<<N * nh, 64, 0, stream>>>(parts, tiles, gate, ldg, (float*)out, ldo, nh, dv, out_scale);
        else
            talk_merge_kernel<bf16><<<N * nh, 64, 0, stream>>>(parts, tiles, gate, ldg, (bf16*)out, ldo, nh, dv, out_scale);
    }
    AGAVE_LAUNCH_CHECK("talk_attention");
    return 0;
}

// ------------------------------------------------------------------ gated linear recurrence
// Per sequence and head a state S [dk][dv] of floats (stored [slot][head][dv][dk]: a column's rows lie
// together), advanced token by token:
//     S <- diag(a) S;   u = beta (v - S^T k)  [delta]  or  u = v  [forget gate];   S <- S + k u^T;   o = S^T q
// so the read-out sees the token's own write.  A column of S (one value element) never meets
// another: DS lanes share a column's dk rows (R each), a wave owns 64 / DS columns, and the four
// consumer waves of a workgroup 4 * 64 / DS columns of one head.  Four producer waves make the gates
// of the next TB tokens into the other half of LDS meanwhile (all their loads asked for before the
// first is used), so that the chain from token to token never waits for memory:
//   delta:   q, k: unit vectors per head (x / sqrt(sum x^2 + unit_eps)), q times dk^-1/2; key head of h is
//            h / (nh / nkv);  a = exp(-exp(A_log[h]) * softplus(dt[h][d] + dt_bias[h][d]));  beta = sigmoid(b[h])
//   forget:  q = silu(q);  f = low + (1 - low) sigmoid(f_in + f_bias);  a = f, k = 1 - f
//   ssd:     one decay per head and token: d = softplus(dt[h] + dt_bias[h]) (exact functions, no clamp),
//            a = exp(-exp(A_log[h]) d) for every key channel; k = B and q = C of the head's group h / (nh / nkv), as
//            they come; u = d v; the read-out gets skip[h] v on top
#define REC_DELTA 0
#define REC_FORGET 1
#define REC_SSD 2

struct RecurrenceArgs {
    const float* q; long ldq;          // delta: [N, nkv*dk]; forget: [N, nh*dk]
    const float* k; long ldk;          // delta: keys [N, nkv*dk]; forget: the gate's input [N, nh*dk]
    const float* v; long ldv;          // [N, nh*dv]
    const float* dt; long lddt;        // delta: [N, nh*dk]; ssd: [N, nh]
    const float* b; long ldb;          // delta: [N, nh]
    const float* a_log;                // delta, ssd: [nh]
    const float* dt_bias;              // delta: [nh*dk]; ssd: [nh]
    const float* skip;                 // ssd: [nh]
    const float* low;                  // forget: [nh*dk]
    const float* f_bias;               // forget: [nh*dk] or null
    float* o; long ldo;                // [N, nh*dv]
    float* state;                      // [slots][nh][dv][dk]
    const int* cu; const int* slots;
    int nh, nkv, dk, dv;
    float unit_eps;                    // delta: inside the root of the unit vectors
};

// softplus by the exact functions, for the one step size a head and token has (the state-space form): what it
// is off by is multiplied into every later state
__device__ __forceinline__ float softplus_exact(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// A lane's R rows of its state column, to and from memory: 16 bytes at a time where the column's
// length allows (R is a multiple of 4, so a lane's rows start at a multiple of 4 too).
template <int R> __device__ __forceinline__ void state_load(float (&S)[R], const float* col_ptr, int d0, int dk, bool live) {
    if ((dk & 3) == 0) {
#pragma unroll
        for (int i = 0; i < R; i += 4) {
            float4 x = {0.f, 0.f, 0.f, 0.f};
            if (live && d0 + i < dk) x = *reinterpret_cast<const float4*>(col_ptr + d0 + i);
            S[i] = x.x; S[i + 1] = x.y; S[i + 2] = x.z; S[i + 3] = x.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < R; ++i) S[i] = (live && d0 + i < dk) ? col_ptr[d0 + i] : 0.f;
    }
}
template <int R> __device__ __forceinline__ void state_store(const float (&S)[R], float* col_ptr, int d0, int dk, bool live) {
    if (!live) return;
    if ((dk & 3) == 0) {
#pragma unroll
        for (int i = 0; i < R; i += 4)
            if (d0 + i < dk) *reinterpret_cast<float4*>(col_ptr + d0 + i) = float4{S[i], S[i + 1], S[i + 2], S[i + 3]};
    } else {
#pragma unroll
        for (int i = 0; i < R; ++i)
            if (d0 + i < dk) col_ptr[d0 + i] = S[i];
    }
}

template <int DS> __device__ __forceinline__ float lanes_sum(float v) {
    v += dpp_get<0xB1, 0xF>(0.f, v);          // quad_perm [1,0,3,2]
    v += dpp_get<0x4E, 0xF>(0.f, v);          // quad_perm [2,3,0,1]
    if (DS == 16) {
        v += dpp_get<0x141, 0xF>(0.f, v);     // row_half_mirror
        v += dpp_get<0x140, 0xF>(0.f, v);     // row_mirror
    }
    return v;
}

// A workgroup barrier that waits for this wave's LDS traffic only.  __syncthreads() also waits for every
// load from memory that is on its way, and the producers' loads for the block after next are meant to stay
// on their way across it: with the full barrier every block of 16 tokens cost a round trip to memory.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <int MODE, int DS, int R, int TB>
__global__ __launch_bounds__(512) void gated_recurrence_kernel(RecurrenceArgs A) {
    constexpr int DP = DS * R;                              // padded rows
    constexpr int CW = 64 / DS, CB = 4 * CW;                // columns a wave, a workgroup
    constexpr int NE = (DP + 63) / 64;                      // elements of a row a producer lane holds
    constexpr int PW = 4;                                   // producer waves (behind the four consumer waves)
    constexpr int NT = TB / PW;                             // tokens of a block a producer wave makes
    __shared__ __attribute__((aligned(16))) float sa[2][TB][DP];
    __shared__ __attribute__((aligned(16))) float sk[2][TB][DP];
    __shared__ __attribute__((aligned(16))) float sq[2][TB][DP];
    __shared__ float sv[2][TB][CB];
    __shared__ float sbeta[2][TB];
    __shared__ float skq[2][TB];                            // k . q of a token, for the read-out

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const bool producer = wv >= 4;
    const int h = blockIdx.y, s = blockIdx.z, col0 = blockIdx.x * CB;
    const int dk = A.dk, dv = A.dv;
    const int r0 = A.cu[s], r1 = A.cu[s + 1];
    const int n_blocks = (r1 - r0 + TB - 1) / TB;

    // ---- consumers: their share of the state
    const int ds = lane & (DS - 1), colb = (wv & 3) * CW + lane / DS, col = col0 + colb;
    float* S_g = A.state + (((size_t)A.slots[s] * A.nh + h) * dv + (col < dv ? col : 0)) * dk;
    float S[R];
    if (!producer) state_load<R>(S, S_g, ds * R, dk, col < dv);
    // ---- producers: what does not change from token to token
    const int pw = wv - 4;
    const int kvh = MODE == REC_FORGET ? h : h / (A.nh / A.nkv);
    float c0[NE], c1[NE];                                   // delta: dt_bias, -;  forget: lower bound, the gate's bias
    float ea = 0.f;
    const float skip = MODE == REC_SSD ? A.skip[h] : 0.f;
    if (producer) {
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            const int d = lane + 64 * e, dd = d < dk ? d : dk - 1;
            if (MODE == REC_DELTA) { c0[e] = A.dt_bias[(size_t)h * dk + dd]; c1[e] = 0.f; }
            else if (MODE == REC_SSD) { c0[e] = A.dt_bias[h]; c1[e] = 0.f; }
            else { c0[e] = A.low[(size_t)h * dk + dd]; c1[e] = A.f_bias ? A.f_bias[(size_t)h * dk + dd] : 0.f; }
        }
        if (MODE != REC_FORGET) ea = expf(A.a_log[h]);
    }

    // what a producer wave has asked for and not yet used: the rows of its tokens of one block
    float x0[NT][NE], x1[NT][NE], x2[NT][NE], vv[NT], bb[NT];
    auto ask = [&](int blk) {
        const int tb = r0 + blk * TB;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            int row = tb + pw + PW * t;
            row = row < r1 ? row : r1 - 1;
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                const int d = lane + 64 * e, dd = d < dk ? d : dk - 1;
                if (MODE == REC_DELTA) {
                    x0[t][e] = A.q[(size_t)row * A.ldq + (size_t)kvh * dk + dd];
                    x1[t][e] = A.k[(size_t)row * A.ldk + (size_t)kvh * dk + dd];
                    x2[t][e] = A.dt[(size_t)row * A.lddt + (size_t)h * dk + dd];
                } else if (MODE == REC_SSD) {
                    x0[t][e] = A.q[(size_t)row * A.ldq + (size_t)kvh * dk + dd];
                    x1[t][e] = A.k[(size_t)row * A.ldk + (size_t)kvh * dk + dd];
                    x2[t][e] = 0.f;
                } else {
                    x0[t][e] = A.q[(size_t)row * A.ldq + (size_t)h * dk + dd];
                    x1[t][e] = A.k[(size_t)row * A.ldk + (size_t)h * dk + dd];
                    x2[t][e] = 0.f;
                }
            }
            const int c = col0 + (lane < CB ? lane : 0);
            vv[t] = A.v[(size_t)row * A.ldv + (size_t)h * dv + (c < dv ? c : dv - 1)];
            bb[t] = MODE == REC_DELTA ? A.b[(size_t)row * A.ldb + h] : (MODE == REC_SSD ? A.dt[(size_t)row * A.lddt + h] : 0.f);
        }
    };
    auto make = [&](int blk, int buf) {
        const int left = r1 - (r0 + blk * TB);              // tokens of this block
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int tt = pw + PW * t;
            if (tt >= left) continue;                       // behind the sequence's end: nobody reads that row
            const bool real = true;
            float qi = 1.f, ki = 1.f;
            if (MODE == REC_DELTA) {
                float qq = 0.f, kk = 0.f;
#pragma unroll
                for (int e = 0; e < NE; ++e)
                    if (lane + 64 * e < dk) { qq = fmaf(x0[t][e], x0[t][e], qq); kk = fmaf(x1[t][e], x1[t][e], kk); }
                qq = wave_sum(qq);
                kk = wave_sum(kk);
                qi = 1.0f / sqrtf(qq + A.unit_eps) / sqrtf((float)dk);
                ki = 1.0f / sqrtf(kk + A.unit_eps);
            }
            float step = 0.f, step_decay = 1.f;             // ssd: the token's step size and what it leaves of the state
            if (MODE == REC_SSD) {
                step = softplus_exact(bb[t] + c0[0]);
                step_decay = expf(-ea * step);
            }
            float kq = 0.f;
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                const int d = lane + 64 * e;
                float a = real ? 0.f : 1.f, kx = 0.f, qx = 0.f;
                if (d < dk && real) {
                    if (MODE == REC_DELTA) {
                        a = decay_f(ea, x2[t][e] + c0[e]);
                        kx = x1[t][e] * ki;
                        qx = x0[t][e] * qi;
                    } else if (MODE == REC_SSD) {
                        a = step_decay;
                        kx = x1[t][e];
                        qx = x0[t][e];
                    } else {
                        const float f = c0[e] + (1.f - c0[e]) * sigmoid_f(x1[t][e] + c1[e]);
                        a = f;
                        kx = 1.f - f;
                        qx = silu_f(x0[t][e]);
                    }
                }
                kq = fmaf(kx, qx, kq);
                if (d < DP) { sa[buf][tt][d] = a; sk[buf][tt][d] = kx; sq[buf][tt][d] = qx; }
            }
            kq = wave_sum(kq);
            if (lane < CB) sv[buf][tt][lane] = real ? vv[t] : 0.f;
            if (lane == 0) {
                sbeta[buf][tt] = (MODE == REC_DELTA && real) ? sigmoid_f(bb[t]) : (MODE == REC_SSD ? step : (real ? 1.f : 0.f));
                skq[buf][tt] = kq;
            }
        }
    };

    // Consumers.  With t = diag(a) S:  S^T k = sum t k,  and the read-out of the new state is
    // sum t q + u (k . q), so both sums run side by side, one round of cross-lane adds serves both, and
    // the state's update S = t + k u is all that the next token waits for.
    auto token = [&](int tb, int buf, int tt) {
        const float4* a4 = reinterpret_cast<const float4*>(&sa[buf][tt][ds * R]);
        const float4* k4 = reinterpret_cast<const float4*>(&sk[buf][tt][ds * R]);
        const float4* q4 = reinterpret_cast<const float4*>(&sq[buf][tt][ds * R]);
        float kreg[R];
        float dk0 = 0.f, dk1 = 0.f, dq0 = 0.f, dq1 = 0.f;
#pragma unroll
        for (int i = 0; i < R / 4; ++i) {
            const float4 a = a4[i], k = k4[i], qv = q4[i];
            kreg[4 * i] = k.x; kreg[4 * i + 1] = k.y; kreg[4 * i + 2] = k.z; kreg[4 * i + 3] = k.w;
            S[4 * i] *= a.x; S[4 * i + 1] *= a.y; S[4 * i + 2] *= a.z; S[4 * i + 3] *= a.w;
            dq0 = fmaf(S[4 * i], qv.x, dq0); dq1 = fmaf(S[4 * i + 1], qv.y, dq1);
            dq0 = fmaf(S[4 * i + 2], qv.z, dq0); dq1 = fmaf(S[4 * i + 3], qv.w, dq1);
            if (MODE == REC_DELTA) {
                dk0 = fmaf(S[4 * i], k.x, dk0); dk1 = fmaf(S[4 * i + 1], k.y, dk1);
                dk0 = fmaf(S[4 * i + 2], k.z, dk0); dk1 = fmaf(S[4 * i + 3], k.w, dk1);
            }
        }
        float u = sv[buf][tt][colb];
        float dq = dq0 + dq1;
        if (MODE == REC_DELTA) {
            float dkk = dk0 + dk1;
            dkk += dpp_get<0xB1, 0xF>(0.f, dkk); dq += dpp_get<0xB1, 0xF>(0.f, dq);
            dkk += dpp_get<0x4E, 0xF>(0.f, dkk); dq += dpp_get<0x4E, 0xF>(0.f, dq);
            if (DS == 16) {
                dkk += dpp_get<0x141, 0xF>(0.f, dkk); dq += dpp_get<0x141, 0xF>(0.f, dq);
                dkk += dpp_get<0x140, 0xF>(0.f, dkk); dq += dpp_get<0x140, 0xF>(0.f, dq);
            }
            u = sbeta[buf][tt] * (u - dkk);
        } else {
            dq = lanes_sum<DS>(dq);
        }
        const float v_in = u;
        if (MODE == REC_SSD) u *= sbeta[buf][tt];
#pragma unroll
        for (int i = 0; i < R; ++i) S[i] = fmaf(kreg[i], u, S[i]);
        float o = fmaf(u, skq[buf][tt], dq);
        if (MODE == REC_SSD) o = fmaf(skip, v_in, o);
        if (ds == 0 && col < dv) A.o[(size_t)(tb + tt) * A.ldo + (size_t)h * dv + col] = o;
    };
    auto consume = [&](int blk, int buf) {
        const int tb = r0 + blk * TB;
        const int nt = r1 - tb;
        if (nt >= TB) {                                     // a whole block: its tokens written out one after another
#pragma unroll
            for (int tt = 0; tt < TB; ++tt) token(tb, buf, tt);
        } else {                                            // the sequence's last tokens (a decode step: one)
            for (int tt = 0; tt < nt; ++tt) token(tb, buf, tt);
        }
    };

    // producers run two blocks ahead with their loads and one with their gates
    if (producer) {
        ask(0);
        make(0, 0);
        if (n_blocks > 1) ask(1);
    }
    lds_barrier();
    for (int blk = 0; blk < n_blocks; ++blk) {
        if (producer) {
            if (blk + 1 < n_blocks) {
                make(blk + 1, (blk + 1) & 1);
                if (blk + 2 < n_blocks) ask(blk + 2);
            }
        } else {
            consume(blk, blk & 1);
        }
        lds_barrier();                                      // the block just read may be overwritten, the one just made be read
    }
    if (!producer) state_store<R>(S, S_g, ds * R, dk, col < dv);
}

// One token per sequence (a decode step): four waves, each with 64 / DS columns, and every wave makes
// the token's gates for itself, so nothing waits for another wave's work and a compute unit holds eight
// such workgroups (the kernel above, with its eight waves and two halves of LDS, holds far fewer).
template <int MODE, int DS, int R>
__global__ __launch_bounds__(256) void gated_recurrence_step_kernel(RecurrenceArgs A) {
    constexpr int DP = DS * R, CW = 64 / DS, CB = 4 * CW, NE = (DP + 63) / 64;
    __shared__ __attribute__((aligned(16))) float sa[4][DP];
    __shared__ __attribute__((aligned(16))) float sk[4][DP];
    __shared__ __attribute__((aligned(16))) float sq[4][DP];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int h = blockIdx.y, s = blockIdx.z, col0 = blockIdx.x * CB;
    const int dk = A.dk, dv = A.dv;
    const size_t row = (size_t)A.cu[s];
    const int ds = lane & (DS - 1), col = col0 + wv * CW + lane / DS;
    float* S_g = A.state + (((size_t)A.slots[s] * A.nh + h) * dv + (col < dv ? col : 0)) * dk;
    float S[R];
    state_load<R>(S, S_g, ds * R, dk, col < dv);
    const int kvh = MODE == REC_FORGET ? h : h / (A.nh / A.nkv);
    float x0[NE], x1[NE], x2[NE], c0[NE], c1[NE];
#pragma unroll
    for (int e = 0; e < NE; ++e) {                          // every load first
        const int d = lane + 64 * e, dd = d < dk ? d : dk - 1;
        if (MODE == REC_DELTA) {
            x0[e] = A.q[row * A.ldq + (size_t)kvh * dk + dd];
            x1[e] = A.k[row * A.ldk + (size_t)kvh * dk + dd];
            x2[e] = A.dt[row * A.lddt + (size_t)h * dk + dd];
            c0[e] = A.dt_bias[(size_t)h * dk + dd];
            c1[e] = 0.f;
        } else if (MODE == REC_SSD) {
            x0[e] = A.q[row * A.ldq + (size_t)kvh * dk + dd];
            x1[e] = A.k[row * A.ldk + (size_t)kvh * dk + dd];
            x2[e] = 0.f;
            c0[e] = c1[e] = 0.f;
        } else {
            x0[e] = A.q[row * A.ldq + (size_t)h * dk + dd];
            x1[e] = A.k[row * A.ldk + (size_t)h * dk + dd];
            x2[e] = 0.f;
            c0[e] = A.low[(size_t)h * dk + dd];
            c1[e] = A.f_bias ? A.f_bias[(size_t)h * dk + dd] : 0.f;
        }
    }
    float u = A.v[row * A.ldv + (size_t)h * dv + (col < dv ? col : dv - 1)];
    float beta = 1.f, ea = 0.f;
    if (MODE == REC_DELTA) {
        beta = sigmoid_f(A.b[row * A.ldb + h]);
        ea = expf(A.a_log[h]);
    }
    float step = 0.f, step_decay = 1.f, skip = 0.f;
    const float v_in = u;
    if (MODE == REC_SSD) {
        step = softplus_exact(A.dt[row * A.lddt + h] + A.dt_bias[h]);
        step_decay = expf(-expf(A.a_log[h]) * step);
        skip = A.skip[h];
        u *= step;
    }
    float qi = 1.f, ki = 1.f;
    if (MODE == REC_DELTA) {
        float qq = 0.f, kk = 0.f;
#pragma unroll
        for (int e = 0; e < NE; ++e)
            if (lane + 64 * e < dk) { qq = fmaf(x0[e], x0[e], qq); kk = fmaf(x1[e], x1[e], kk); }
        qq = wave_sum(qq);
        kk = wave_sum(kk);
        qi = 1.0f / sqrtf(qq + A.unit_eps) / sqrtf((float)dk);
        ki = 1.0f / sqrtf(kk + A.unit_eps);
    }
    float kq = 0.f;
#pragma unroll
    for (int e = 0; e < NE; ++e) {
        const int d = lane + 64 * e;
        float a = 0.f, kx = 0.f, qx = 0.f;
        if (d < dk) {
            if (MODE == REC_DELTA) {
                a = decay_f(ea, x2[e] + c0[e]);
                kx = x1[e] * ki;
                qx = x0[e] * qi;
            } else if (MODE == REC_SSD) {
                a = step_decay;
                kx = x1[e];
                qx = x0[e];
            } else {
                const float f = c0[e] + (1.f - c0[e]) * sigmoid_f(x1[e] + c1[e]);
                a = f;
                kx = 1.f - f;
                qx = silu_f(x0[e]);
            }
        }
        kq = fmaf(kx, qx, kq);
        if (d < DP) { sa[wv][d] = a; sk[wv][d] = kx; sq[wv][d] = qx; }
    }
    kq = wave_sum(kq);
    __syncthreads();                                        // (a wave reads only what it wrote itself)
    float dkk = 0.f, dq = 0.f;
    float kreg[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int d = ds * R + i;
        kreg[i] = sk[wv][d];
        S[i] *= sa[wv][d];
        dq = fmaf(S[i], sq[wv][d], dq);
        if (MODE == REC_DELTA) dkk = fmaf(S[i], kreg[i], dkk);
    }
    dq = lanes_sum<DS>(dq);
    if (MODE == REC_DELTA) u = beta * (u - lanes_sum<DS>(dkk));
#pragma unroll
    for (int i = 0; i < R; ++i) S[i] = fmaf(kreg[i], u, S[i]);
    state_store<R>(S, S_g, ds * R, dk, col < dv);
    if (ds == 0 && col < dv) A.o[row * A.ldo + (size_t)h * dv + col] = fmaf(u, kq, dq) + skip * v_in;
}

template <int MODE>
static int launch_recurrence_step(const RecurrenceArgs& A, int n_seqs, hipStream_t stream) {
    const int cb = A.dk <= 32 ? 64 : 16;
    const dim3 grid((A.dv + cb - 1) / cb, A.nh, n_seqs);
    if (A.dk <= 32) gated_recurrence_step_kernel<MODE, 4, 8><<<grid, 256, 0, stream>>>(A);
    else if (A.dk <= 64) gated_recurrence_step_kernel<MODE, 16, 4><<<grid, 256, 0, stream>>>(A);
    else if (A.dk <= 128) gated_recurrence_step_kernel<MODE, 16, 8><<<grid, 256, 0, stream>>>(A);
    else gated_recurrence_step_kernel<MODE, 16, 16><<<grid, 256, 0, stream>>>(A);
    AGAVE_LAUNCH_CHECK("gated_recurrence_step");
    return 0;
}

template <int MODE>
static int launch_recurrence(const RecurrenceArgs& A, int n_seqs, hipStream_t stream) {
    // (for a decode step, 64 columns a workgroup with four lanes a column were measured too: a head's gates
    // are then made twice instead of eight times, and the step was 6 % slower: the longer chain of a token)
    const int cb = A.dk <= 32 ? 64 : 16;                    // columns a workgroup, as the kernel's CB
    const dim3 grid((A.dv + cb - 1) / cb, A.nh, n_seqs);
    if (A.dk <= 32) gated_recurrence_kernel<MODE, 4, 8, 16><<<grid, 512, 0, stream>>>(A);
    else if (A.dk <= 64) gated_recurrence_kernel<MODE, 16, 4, 16><<<grid, 512, 0, stream>>>(A);
    else if (A.dk <= 128) gated_recurrence_kernel<MODE, 16, 8, 16><<<grid, 512, 0, stream>>>(A);
    else gated_recurrence_kernel<MODE, 16, 16, 8><<<grid, 512, 0, stream>>>(A);
    AGAVE_LAUNCH_CHECK("gated_recurrence");
    return 0;
}

extern "C" int agave_gated_recurrence(int mode, const float* q, long ldq, const float* k, long ldk, const float* v, long ldv,
                                      const float* dt, long lddt, const float* b, long ldb, const float* a_log,
                                      const float* dt_bias, const float* low, const float* f_bias, const float* skip, float* o, long ldo,
                                      float* state, const int* cu, const int* slots, int n_seqs, int nh, int nkv, int dk,
                                      int dv, float unit_eps, int one_token_each, hipStream_t stream) {
    AGAVE_CHECK(mode == REC_DELTA || mode == REC_FORGET || mode == REC_SSD, "gated_recurrence: unknown mode %d", mode);
    AGAVE_CHECK(n_seqs >= 0 && nh > 0 && nkv > 0 && dk > 0 && dv > 0, "gated_recurrence: bad sizes B=%d nh=%d nkv=%d dk=%d dv=%d", n_seqs, nh, nkv, dk, dv);
    AGAVE_CHECK(dk <= 256, "gated_recurrence: %d key channels a head (up to 256 are supported)", dk);
    AGAVE_CHECK(nh % nkv == 0, "gated_recurrence: %d heads are not a multiple of %d key heads", nh, nkv);
    AGAVE_CHECK(q && k && v && o && state && cu && slots, "gated_recurrence: null buffer");
    AGAVE_CHECK(ldv >= (long)nh * dv && ldo >= (long)nh * dv, "gated_recurrence: a row stride is too small");
    AGAVE_CHECK(n_seqs < 65536 && nh < 65536, "gated_recurrence: too many sequences or heads");
    if (mode == REC_DELTA) {
        AGAVE_CHECK(dt && b && a_log && dt_bias, "gated_recurrence: the delta rule needs dt, b, A_log and dt_bias");
        AGAVE_CHECK(ldq >= (long)nkv * dk && ldk >= (long)nkv * dk && lddt >= (long)nh * dk && ldb >= nh, "gated_recurrence: a row stride is too small");
    } else if (mode == REC_SSD) {
        AGAVE_CHECK(dt && a_log && dt_bias && skip, "gated_recurrence: the state-space form needs dt, A_log, dt_bias and the skip weights");
        AGAVE_CHECK(ldq >= (long)nkv * dk && ldk >= (long)nkv * dk && lddt >= nh, "gated_recurrence: a row stride is too small");
    } else {
        AGAVE_CHECK(low, "gated_recurrence: the forget gate needs its lower bound");
        AGAVE_CHECK(nkv == nh && ldq >= (long)nh * dk && ldk >= (long)nh * dk, "gated_recurrence: the forget-gate form has a gate per head");
    }
    if (n_seqs == 0) return 0;
    RecurrenceArgs A{q, ldq, k, ldk, v, ldv, dt, lddt, b, ldb, a_log, dt_bias, skip, low, f_bias, o, ldo, state, cu, slots, nh, nkv, dk, dv, unit_eps};
    if (one_token_each) {                                   // the host vouches that every sequence brings one token
        if (mode == REC_SSD) return launch_recurrence_step<REC_SSD>(A, n_seqs, stream);
        return mode == REC_DELTA ? launch_recurrence_step<REC_DELTA>(A, n_seqs, stream) : launch_recurrence_step<REC_FORGET>(A, n_seqs, stream);
    }
    if (mode == REC_SSD) return launch_recurrence<REC_SSD>(A, n_seqs, stream);
    return mode == REC_DELTA ? launch_recurrence<REC_DELTA>(A, n_seqs, stream) : launch_recurrence<REC_FORGET>(A, n_seqs, stream);
}

// ------------------------------------------------------------------ read-out norm with a gate
//   out[t][h][e] = o[t][h][e] * rsqrt(mean_e(o[t][h]^2) + eps) * w[e] * (gate ? sigmoid(gate[t][h][e]) : 1) * out_scale
template <typename T>
__global__ __launch_bounds__(64) void head_norm_gate_kernel(const float* __restrict__ o, long ldo_in, const float* __restrict__ w,
                                                            const float* __restrict__ gate, long ldg, T* __restrict__ out,
                                                            long ldo, int nh, int dv, float eps, float out_scale) {
    const int t = blockIdx.x / nh, h = blockIdx.x % nh, lane = threadIdx.x;
    const float* x = o + (size_t)t * ldo_in + (size_t)h * dv;
    float ss = 0.f;
    for (int e = lane; e < dv; e += 64) ss = fmaf(x[e], x[e], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
    for (int e = lane; e < dv; e += 64) {
        float y = x[e] * inv * w[e];
        if (gate) y *= sigmoid_f(gate[(size_t)t * ldg + (size_t)h * dv + e]);
        st(out + (size_t)t * ldo + (size_t)h * dv + e, y * out_scale);
    }
}

extern "C" int agave_head_norm_gate(int dtype, const float* o, long ldo_in, const float* w, const float* gate, long ldg,
                                    void* out, long ldo, int N, int nh, int dv, float eps, float out_scale, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && nh > 0 && dv > 0, "head_norm_gate: bad sizes N=%d nh=%d dv=%d", N, nh, dv);
    AGAVE_CHECK(o && w && out && ldo_in >= (long)nh * dv && ldo >= (long)nh * dv && (!gate || ldg >= (long)nh * dv), "head_norm_gate: bad buffers");
    AGAVE_CHECK((long)N * nh < 2147483647L, "head_norm_gate: too many rows");
    if (N == 0) return 0;
    if (dtype == AGAVE_F32)
        head_norm_gate_kernel<float><<<N * nh, 64, 0, stream>>>(o, ldo_in, w, gate, ldg, (float*)out, ldo, nh, dv, eps, out_scale);
    else if (dtype == AGAVE_BF16)
        head_norm_gate_kernel<bf16><<<N * nh, 64, 0, stream>>>(o, ldo_in, w, gate, ldg, (bf16*)out, ldo, nh, dv, eps, out_scale);
    else
        AGAVE_CHECK(false, "head_norm_gate: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("head_norm_gate");
    return 0;
}

// ------------------------------------------------------------------ a gate, then a norm in equal parts of the row
//   g = y * silu(z);  out = g / sqrt(mean over the part (g^2) + eps) * w     (w is [parts * size])
// A workgroup per (token, part), of one to four waves by the part's size; a thread keeps up to sixteen gated values in
// registers between the sum of squares and the output (longer parts are computed twice).
template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* __restrict__ y, long ldy, const float* __restrict__ z,
                                                               long ldz, const float* __restrict__ w, T* __restrict__ out, long ldo,
                                                               int parts, int size, float eps) {
    __shared__ float red[8];
    constexpr int KEEP = 16;
    const int t = blockIdx.x / parts, g = blockIdx.x % parts, tid = threadIdx.x, nt = blockDim.x;
    const float* yr = y + (size_t)t * ldy + (size_t)g * size;
    const float* zr = z + (size_t)t * ldz + (size_t)g * size;
    const float* wr = w + (size_t)g * size;
    float yv[KEEP], zv[KEEP], gv[KEEP];
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {                    // (loads from inside the part, emptied afterwards)
        const int e = tid + i * nt;
        yv[i] = yr[e < size ? e : 0];
        zv[i] = zr[e < size ? e : 0];
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
        gv[i] = tid + i * nt < size ? yv[i] * (zv[i] / (1.0f + expf(-zv[i]))) : 0.f;
        ss = fmaf(gv[i], gv[i], ss);
    }
    for (int e = tid + KEEP * nt; e < size; e += nt) {
        const float zz = zr[e], v = yr[e] * (zz / (1.0f + expf(-zz)));
        ss = fmaf(v, v, ss);
    }
    ss = nt > 64 ? block_sum(ss, red) : wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)size + eps);
    T* o = out + (size_t)t * ldo + (size_t)g * size;
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
        const int e = tid + i * nt;
        if (e < size) st(o + e, gv[i] * inv * wr[e]);
    }
    for (int e = tid + KEEP * nt; e < size; e += nt) {
        const float zz = zr[e], v = yr[e] * (zz / (1.0f + expf(-zz)));
        st(o + e, v * inv * wr[e]);
    }
}

extern "C" int agave_gated_group_norm(int dtype, const float* y, long ldy, const float* z, long ldz, const float* w, void* out,
                                      long ldo, int N, int parts, int size, float eps, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && parts > 0 && size > 0, "gated_group_norm: bad sizes N=%d parts=%d size=%d", N, parts, size);
    const long width = (long)parts * size;
    AGAVE_CHECK(y && z && w && out && ldy >= width && ldz >= width && ldo >= width, "gated_group_norm: bad buffers");
    AGAVE_CHECK((long)N * parts < 2147483647L, "gated_group_norm: too many rows");
    if (N == 0) return 0;
    const int threads = size <= 256 ? 64 : size <= 1024 ? 128 : 256;
    if (dtype == AGAVE_F32)
        gated_group_norm_kernel<float><<<N * parts, threads, 0, stream>>>(y, ldy, z, ldz, w, (float*)out, ldo, parts, size, eps);
    else if (dtype == AGAVE_BF16)
        gated_group_norm_kernel<bf16><<<N * parts, threads, 0, stream>>>(y, ldy, z, ldz, w, (bf16*)out, ldo, parts, size, eps);
    else
        AGAVE_CHECK(false, "gated_group_norm: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("gated_group_norm");
    return 0;
}

// ------------------------------------------------------------------ a weighted sum of two branches
//   out = sa * a + sb * b, summed in 32-bit (for mixers that run side by side and cannot share an output product)
template <typename T>
__global__ void scaled_sum_kernel(const T* __restrict__ a, long lda, float sa, const T* __restrict__ b, long ldb, float sb,
                                  T* __restrict__ out, long ldo, long total, int cols) {
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const long r = idx / cols;
        const int c = (int)(idx % cols);
        st(out + r * ldo + c, sa * ld(a + r * lda + c) + sb * ld(b + r * ldb + c));
    }
}

extern "C" int agave_scaled_sum(int dtype, const void* a, long lda, float sa, const void* b, long ldb, float sb, void* out,
                                long ldo, int rows, int cols, hipStream_t stream) {
    AGAVE_CHECK(rows >= 0 && cols > 0 && lda >= cols && ldb >= cols && ldo >= cols, "scaled_sum: bad sizes rows=%d cols=%d", rows, cols);
    AGAVE_CHECK(a && b && out, "scaled_sum: null buffer");
    if (rows == 0) return 0;
    const long total = (long)rows * cols;
    long blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == AGAVE_F32)
        scaled_sum_kernel<float><<<(int)blocks, 256, 0, stream>>>((const float*)a, lda, sa, (const float*)b, ldb, sb, (float*)out, ldo, total, cols);
    else if (dtype == AGAVE_BF16)
        scaled_sum_kernel<bf16><<<(int)blocks, 256, 0, stream>>>((const bf16*)a, lda, sa, (const bf16*)b, ldb, sb, (bf16*)out, ldo, total, cols);
    else
        AGAVE_CHECK(false, "scaled_sum: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("scaled_sum");
    return 0;
}
