// A gated linear recurrence per channel (the recurrent unit of Griffin's recurrent block) for gfx950.
//
//   r = sigmoid(A_r[b] u_b + b_r[b]),  g = sigmoid(A_i[b] u_b + b_i[b])      in each of `blocks` equal parts b of the channels
//   log a = -decay r        (decay = c softplus(lam), made once on the host)
//   S <- a S + sqrt(1 - a^2) g u          out = S gelu_tanh(y)
//
// rglru_gates: the two block-diagonal products and everything up to (a, sqrt(1 - a^2) g u), in 32-bit whatever the
// element type of the gate matrices.  A workgroup takes 32 tokens x 64 channels of a block; the inputs and both
// matrices' tiles pass through LDS in steps of 32 along the block.  Steps of few tokens and bfloat16 matrices with
// blocks the matrix cores take have kernels of their own (below).
// rglru_scan: S_t = a_t S_(t-1) + x_t along each sequence, over the step's rows in chunks: a chunk's effect on what
// comes in is (P, Q) with S_end = P S_in + Q (summarise), the chunks' carries follow one after another (carry), then
// every chunk runs again from its carry and writes the rows (apply).  A sequence's first row of the step starts from
// the sequence's state, its last row leaves the state.  Steps of few rows are one chunk and one launch.
#include "common_impl.h"
#include "mfma.h"
#include <math.h>

#define GT 32          // tokens a workgroup
#define GO 64          // channels a workgroup
#define GK 32          // step along the block

template <typename T>
__global__ __launch_bounds__(256) void rglru_gates_kernel(const float* __restrict__ u, long ldu, const T* __restrict__ wr,
                                                          const T* __restrict__ wi, const float* __restrict__ br,
                                                          const float* __restrict__ bi, const float* __restrict__ decay,
                                                          float* __restrict__ a_out, float* __restrict__ x_out, int N, int W,
                                                          int bw) {
    __shared__ float us[GT][GK + 1];
    __shared__ float rs[GO][GK + 1];
    __shared__ float is[GO][GK + 1];
    const int t0 = blockIdx.x * GT, b = blockIdx.y, o0 = blockIdx.z * GO;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;          // channel o0 + tx, tokens t0 + ty + 4 i
    float ar[GT / 4], ai[GT / 4];
#pragma unroll
    for (int i = 0; i < GT / 4; ++i) ar[i] = ai[i] = 0.f;
    const T* wrb = wr + (size_t)b * bw * bw;
    const T* wib = wi + (size_t)b * bw * bw;
    for (int k0 = 0; k0 < bw; k0 += GK) {
        for (int i = threadIdx.x; i < GT * GK; i += 256) {
            const int r = i / GK, k = i % GK;
            us[r][k] = (t0 + r < N && k0 + k < bw) ? u[(size_t)(t0 + r) * ldu + (size_t)b * bw + k0 + k] : 0.f;
        }
        for (int i = threadIdx.x; i < GO * GK; i += 256) {
            const int r = i / GK, k = i % GK;
            const bool in = o0 + r < bw && k0 + k < bw;
            rs[r][k] = in ? ld(wrb + (size_t)(o0 + r) * bw + k0 + k) : 0.f;
            is[r][k] = in ? ld(wib + (size_t)(o0 + r) * bw + k0 + k) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int k = 0; k < GK; ++k) {
            const float a = rs[tx][k], c = is[tx][k];
#pragma unroll
            for (int i = 0; i < GT / 4; ++i) {
                const float x = us[ty + 4 * i][k];
                ar[i] = fmaf(a, x, ar[i]);
                ai[i] = fmaf(c, x, ai[i]);
            }
        }
        __syncthreads();
    }
    const int o = o0 + tx;
    if (o >= bw) return;
    const int ch = b * bw + o;
    const float rb = br[ch], ib = bi[ch], dc = decay[ch];
#pragma unroll
    for (int i = 0; i < GT / 4; ++i) {
        const int t = t0 + ty + 4 * i;
        if (t >= N) continue;
        const float r = 1.0f / (1.0f + expf(-(ar[i] + rb)));
        const float g = 1.0f / (1.0f + expf(-(ai[i] + ib)));
        const float log_a = -dc * r;
        const float a = expf(log_a);
        const float m = sqrtf(fmaxf(-expm1f(2.0f * log_a), 0.f));        // sqrt(1 - a^2), exact where a is near 1
        a_out[(size_t)t * W + ch] = a;
        x_out[(size_t)t * W + ch] = m * g * u[(size_t)t * ldu + ch];
    }
}

// The same for steps of few tokens (decode steps): a wave per channel, the lanes along the block's inputs, sixteen
// (or eight) tokens at a time; the gate matrices' rows stream once, nothing waits in LDS, no load stands under a condition.
template <typename T, int NT>
__global__ __launch_bounds__(256) void rglru_gates_few_kernel(const float* __restrict__ u, long ldu, const T* __restrict__ wr,
                                                              const T* __restrict__ wi, const float* __restrict__ br,
                                                              const float* __restrict__ bi, const float* __restrict__ decay,
                                                              float* __restrict__ a_out, float* __restrict__ x_out, int N, int W,
                                                              int bw) {
    const int lane = threadIdx.x & 63, ch = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (ch >= W) return;
    const int b = ch / bw, o = ch % bw;
    const T* wrr = wr + ((size_t)b * bw + o) * bw;
    const T* wir = wi + ((size_t)b * bw + o) * bw;
    const float rb = br[ch], ib = bi[ch], dc = decay[ch];
    for (int t0 = 0; t0 < N; t0 += NT) {
        float ar[NT], ai[NT];
#pragma unroll
        for (int i = 0; i < NT; ++i) ar[i] = ai[i] = 0.f;
        for (int k0 = 0; k0 < bw; k0 += 64) {
            const int k = k0 + lane < bw ? k0 + lane : bw - 1;
            const float live = k0 + lane < bw ? 1.f : 0.f;
            const float a = ld(wrr + k) * live, c = ld(wir + k) * live;
#pragma unroll
            for (int i = 0; i < NT; ++i) {
                const float x = u[(size_t)(t0 + i < N ? t0 + i : N - 1) * ldu + (size_t)b * bw + k];
                ar[i] = fmaf(a, x, ar[i]);
                ai[i] = fmaf(c, x, ai[i]);
            }
        }
        float zr = 0.f, zi = 0.f;
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            const float r = wave_sum(ar[i]), g = wave_sum(ai[i]);
            if (lane == i) {
                zr = r;
                zi = g;
            }
        }
        const int t = t0 + lane;
        if (lane < NT && t < N) {
            const float r = 1.0f / (1.0f + expf(-(zr + rb)));
            const float g = 1.0f / (1.0f + expf(-(zi + ib)));
            const float log_a = -dc * r;
            a_out[(size_t)t * W + ch] = expf(log_a);
            x_out[(size_t)t * W + ch] = sqrtf(fmaxf(-expm1f(2.0f * log_a), 0.f)) * g * u[(size_t)t * ldu + ch];
        }
    }
}

// The same on the matrix cores, for bfloat16 gate matrices and blocks that are a multiple of 32 wide: the 32-bit inputs
// are taken apart into two bfloat16 numbers, u = hi + lo with hi = bf16(u) and lo = bf16(u - hi), and both parts are
// multiplied (what is lost is below 2^-16 of u, and the sums are 32-bit).  A workgroup of four waves takes 64 channels
// x 64 tokens of one block, a wave 16 channels: per step of 32 along the block it reads its two gates' operands
// (16 bytes a lane, straight from the matrices' rows) and four tiles of tokens (32 bytes a lane each).
__global__ __launch_bounds__(256) void rglru_gates_mfma_kernel(const float* __restrict__ u, long ldu, const bf16* __restrict__ wr,
                                                               const bf16* __restrict__ wi, const float* __restrict__ br,
                                                               const float* __restrict__ bi, const float* __restrict__ decay,
                                                               float* __restrict__ a_out, float* __restrict__ x_out, int N, int W,
                                                               int bw) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int t0 = blockIdx.x * 64, b = blockIdx.y, o0 = blockIdx.z * 64 + 16 * w;
    if (o0 >= bw) return;
    const bf16* wrr = wr + ((size_t)b * bw + o0 + c) * bw + 8 * g;
    const bf16* wir = wi + ((size_t)b * bw + o0 + c) * bw + 8 * g;
    const float* urow[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int t = t0 + 16 * j + c;
        urow[j] = u + (size_t)(t < N ? t : N - 1) * ldu + (size_t)b * bw + 8 * g;
    }
    f32x4_t ar[4], ai[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) ar[j] = ai[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < bw; k0 += 32) {
        frag16 fr, fi;
        fr.u = *reinterpret_cast<const uint4*>(wrr + k0);
        fi.u = *reinterpret_cast<const uint4*>(wir + k0);
        float4 lo4[4], hi4[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            lo4[j] = *reinterpret_cast<const float4*>(urow[j] + k0);
            hi4[j] = *reinterpret_cast<const float4*>(urow[j] + k0 + 4);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float x[8] = {lo4[j].x, lo4[j].y, lo4[j].z, lo4[j].w, hi4[j].x, hi4[j].y, hi4[j].z, hi4[j].w};
            frag16 big, small;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t hb = f32x2_to_bf16x2(x[2 * e], x[2 * e + 1]);
                const float h0 = __uint_as_float(hb << 16), h1 = __uint_as_float(hb & 0xffff0000u);
                big.r[e] = hb;
                small.r[e] = f32x2_to_bf16x2(x[2 * e] - h0, x[2 * e + 1] - h1);
            }
            ar[j] = mfma_16x16x32(fr, big, ar[j]);
            ar[j] = mfma_16x16x32(fr, small, ar[j]);
            ai[j] = mfma_16x16x32(fi, big, ai[j]);
            ai[j] = mfma_16x16x32(fi, small, ai[j]);
        }
    }
    // lane holds channels o0 + 4 g .. + 4 of token t0 + 16 j + c
    const int ch = b * bw + o0 + 4 * g;
    const float4 rb = *reinterpret_cast<const float4*>(br + ch), ib = *reinterpret_cast<const float4*>(bi + ch),
                 dc = *reinterpret_cast<const float4*>(decay + ch);
    const float rbv[4] = {rb.x, rb.y, rb.z, rb.w}, ibv[4] = {ib.x, ib.y, ib.z, ib.w}, dcv[4] = {dc.x, dc.y, dc.z, dc.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int t = t0 + 16 * j + c;
        if (t >= N) continue;
        const float4 uv = *reinterpret_cast<const float4*>(u + (size_t)t * ldu + ch);
        const float uu[4] = {uv.x, uv.y, uv.z, uv.w};
        float av[4], xv[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float r = 1.0f / (1.0f + expf(-(ar[j][e] + rbv[e])));
            const float gg = 1.0f / (1.0f + expf(-(ai[j][e] + ibv[e])));
            const float log_a = -dcv[e] * r;
            av[e] = expf(log_a);
            xv[e] = sqrtf(fmaxf(-expm1f(2.0f * log_a), 0.f)) * gg * uu[e];
        }
        *reinterpret_cast<float4*>(a_out + (size_t)t * W + ch) = make_float4(av[0], av[1], av[2], av[3]);
        *reinterpret_cast<float4*>(x_out + (size_t)t * W + ch) = make_float4(xv[0], xv[1], xv[2], xv[3]);
    }
}

extern "C" int agave_rglru_gates(int w_dtype, const float* u, long ldu, const void* wr, const void* wi, const float* br,
                                 const float* bi, const float* decay, float* a_out, float* x_out, int N, int W, int blocks,
                                 hipStream_t stream) {
    AGAVE_CHECK(u && wr && wi && br && bi && decay && a_out && x_out, "rglru_gates: null buffer");
    AGAVE_CHECK(N >= 0 && W > 0 && blocks > 0 && W % blocks == 0 && ldu >= W, "rglru_gates: %d channels in %d blocks, row stride %ld", W, blocks, ldu);
    if (N == 0) return 0;
    const int bw = W / blocks;
    const dim3 grid((N + GT - 1) / GT, blocks, (bw + GO - 1) / GO);
    AGAVE_CHECK(grid.y <= 65535 && grid.z <= 65535, "rglru_gates: too many blocks");
    if (N <= 64) {
        const int blocks = (W + 3) / 4;
#define GATES_FEW(T_, NT_) rglru_gates_few_kernel<T_, NT_><<<blocks, 256, 0, stream>>>(u, ldu, (const T_*)wr, (const T_*)wi, br, bi, decay, a_out, x_out, N, W, bw)
        if (w_dtype == AGAVE_F32) {
            if (N <= 8) GATES_FEW(float, 8); else GATES_FEW(float, 16);
        } else if (w_dtype == AGAVE_BF16) {
            if (N <= 8) GATES_FEW(bf16, 8); else GATES_FEW(bf16, 16);
        }
#undef GATES_FEW
        else
            AGAVE_CHECK(false, "rglru_gates: unknown dtype %d", w_dtype);
        AGAVE_LAUNCH_CHECK("rglru_gates");
        return 0;
    }
    if (w_dtype == AGAVE_BF16 && bw % 32 == 0 && ldu % 4 == 0 && ((uintptr_t)u % 16) == 0 && ((uintptr_t)wr % 16) == 0 &&
        ((uintptr_t)wi % 16) == 0 && ((uintptr_t)br % 16) == 0 && ((uintptr_t)bi % 16) == 0 && ((uintptr_t)decay % 16) == 0 &&
        ((uintptr_t)a_out % 16) == 0 && ((uintptr_t)x_out % 16) == 0) {
        const dim3 mgrid((N + 63) / 64, blocks, (bw + 63) / 64);
        rglru_gates_mfma_kernel<<<mgrid, 256, 0, stream>>>(u, ldu, (const bf16*)wr, (const bf16*)wi, br, bi, decay, a_out, x_out, N, W, bw);
        AGAVE_LAUNCH_CHECK("rglru_gates");
        return 0;
    }
    if (w_dtype == AGAVE_F32)
        rglru_gates_kernel<float><<<grid, 256, 0, stream>>>(u, ldu, (const float*)wr, (const float*)wi, br, bi, decay, a_out, x_out, N, W, bw);
    else if (w_dtype == AGAVE_BF16)
        rglru_gates_kernel<bf16><<<grid, 256, 0, stream>>>(u, ldu, (const bf16*)wr, (const bf16*)wi, br, bi, decay, a_out, x_out, N, W, bw);
    else
        AGAVE_CHECK(false, "rglru_gates: unknown dtype %d", w_dtype);
    AGAVE_LAUNCH_CHECK("rglru_gates");
    return 0;
}

// ------------------------------------------------------------------ the recurrence over a step's rows
struct ScanArgs {
    const float* a; const float* x;                  // [N][W]
    const float* y; long ldy;                        // [N][W] (strided): the other branch before its activation
    const float* y_bias;                             // [W] or null: added before the activation
    void* out; int out_dtype; long ldo;              // [N][W]
    float* state;                                    // [slots][W]
    const int* tok_seq; const int* cu; const int* slots;
    float* P; float* Q; float* carry;                // [chunks][W] each
    float* fin;                                      // [sequences][W]: the last rows' states wait here while other chunks still read the old ones; null: written in place
    int N, W, L;
};

__device__ __forceinline__ float gelu_tanh_f(float z) {
    const float c = 0.7978845608028654f;
    return 0.5f * z * (1.0f + tanhf(c * (z + 0.044715f * z * z * z)));
}

// MODE 0: (P, Q) of chunk blockIdx.y;  MODE 1: the chunk again from its carry, rows and states written.
// Which rows start or end a sequence's part of the step, and the sequences' slots, are looked up once a workgroup
// (a row a thread) and wait in LDS, so that the chain over the rows holds no load that depends on another.
#define SCAN_MAX_L 64
template <int MODE>
__global__ __launch_bounds__(256) void rglru_scan_kernel(ScanArgs A) {
    __shared__ int flags[SCAN_MAX_L], slot_of[SCAN_MAX_L], seq_of[SCAN_MAX_L];
    const int k = blockIdx.y;
    const int t0 = k * A.L, t1 = min(A.N, t0 + A.L);
    if ((int)threadIdx.x < t1 - t0) {
        const int t = t0 + threadIdx.x;
        const int b = A.tok_seq[t];
        flags[threadIdx.x] = (t == A.cu[b] ? 1 : 0) | (t + 1 == A.cu[b + 1] ? 2 : 0);
        slot_of[threadIdx.x] = A.slots[b];
        seq_of[threadIdx.x] = b;
    }
    __syncthreads();
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch >= A.W) return;
    float P = 1.f, S = (MODE == 1 && k > 0 && A.carry) ? A.carry[(size_t)k * A.W + ch] : 0.f;
    const float yb = (MODE == 1 && A.y_bias) ? A.y_bias[ch] : 0.f;
#pragma unroll 4
    for (int t = t0; t < t1; ++t) {
        const int f = flags[t - t0];
        const float a = A.a[(size_t)t * A.W + ch], x = A.x[(size_t)t * A.W + ch];
        float y = 0.f;
        if (MODE == 1) y = A.y[(size_t)t * A.ldy + ch] + yb;
        if (f & 1) {
            S = A.state[(size_t)slot_of[t - t0] * A.W + ch];
            P = 0.f;
        }
        S = fmaf(a, S, x);
        P *= a;
        if (MODE == 1) {
            const float v = S * gelu_tanh_f(y);
            if (A.out_dtype == AGAVE_F32) ((float*)A.out)[(size_t)t * A.ldo + ch] = v;
            else ((bf16*)A.out)[(size_t)t * A.ldo + ch] = f32_to_bf16(v);
            if (f & 2) {
                if (A.fin) A.fin[(size_t)seq_of[t - t0] * A.W + ch] = S;
                else A.state[(size_t)slot_of[t - t0] * A.W + ch] = S;
            }
        }
    }
    if (MODE == 0) {
        A.P[(size_t)k * A.W + ch] = P;
        A.Q[(size_t)k * A.W + ch] = S;
    }
}

// carry[k] = what enters chunk k: carry[k + 1] = P[k] carry[k] + Q[k] (chunk 0 always starts at a sequence's first row)
__global__ __launch_bounds__(64) void rglru_carry_kernel(ScanArgs A, int chunks) {
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch >= A.W) return;
    float S = 0.f;
    int k = 0;
    for (; k + 8 < chunks; k += 8) {                   // eight chunks' (P, Q) asked for at once, then the chain
        float p[8], q[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            p[i] = A.P[(size_t)(k + i) * A.W + ch];
            q[i] = A.Q[(size_t)(k + i) * A.W + ch];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            S = fmaf(p[i], S, q[i]);
            A.carry[(size_t)(k + i + 1) * A.W + ch] = S;
        }
    }
    for (; k + 1 < chunks; ++k) {
        S = fmaf(A.P[(size_t)k * A.W + ch], S, A.Q[(size_t)k * A.W + ch]);
        A.carry[(size_t)(k + 1) * A.W + ch] = S;
    }
}

__global__ __launch_bounds__(256) void rglru_states_kernel(ScanArgs A) {
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch < A.W) A.state[(size_t)A.slots[blockIdx.y] * A.W + ch] = A.fin[(size_t)blockIdx.y * A.W + ch];
}

extern "C" int agave_rglru_scan(const float* a, const float* x, const float* y, long ldy, const float* y_bias, void* out, int out_dtype, long ldo,
                                float* state, const int* tok_seq, const int* cu, const int* slots, float* scratch,
                                long scratch_floats, int N, int n_seqs, int W, int L, int one_row_each, hipStream_t stream) {
    AGAVE_CHECK(a && x && y && out && state && tok_seq && cu && slots, "rglru_scan: null buffer");
    AGAVE_CHECK(N >= 0 && W > 0 && L > 0 && L <= SCAN_MAX_L && ldy >= W && ldo >= W, "rglru_scan: bad sizes N=%d W=%d L=%d", N, W, L);
    AGAVE_CHECK(out_dtype == AGAVE_F32 || out_dtype == AGAVE_BF16, "rglru_scan: unknown dtype %d", out_dtype);
    if (N == 0) return 0;
    if (one_row_each) {
        // every row is a sequence's first and last of the step: a chunk a row, each from its slot's state and back to it
        AGAVE_CHECK(N == n_seqs && N <= 65535, "rglru_scan: a step of one row a sequence has as many rows as sequences");
        ScanArgs E{a, x, y, ldy, y_bias, out, out_dtype, ldo, state, tok_seq, cu, slots, nullptr, nullptr, nullptr, nullptr, N, W, 1};
        rglru_scan_kernel<1><<<dim3((W + 255) / 256, N), 256, 0, stream>>>(E);
        AGAVE_LAUNCH_CHECK("rglru_scan");
        return 0;
    }
    const int chunks = (N + L - 1) / L;
    AGAVE_CHECK(chunks <= 65535, "rglru_scan: %d chunks of rows", chunks);
    ScanArgs A{a, x, y, ldy, y_bias, out, out_dtype, ldo, state, tok_seq, cu, slots, nullptr, nullptr, nullptr, nullptr, N, W, L};
    const dim3 grid((W + 255) / 256, chunks);
    if (chunks > 1) {
        const long need = (3L * chunks + n_seqs) * W;
        AGAVE_CHECK(n_seqs > 0 && n_seqs <= 65535 && scratch && scratch_floats >= need, "rglru_scan: %d chunks and %d sequences need %ld floats of scratch", chunks, n_seqs, need);
        A.fin = scratch + 3 * (size_t)chunks * W;
        A.P = scratch;
        A.Q = scratch + (size_t)chunks * W;
        A.carry = scratch + 2 * (size_t)chunks * W;
        rglru_scan_kernel<0><<<grid, 256, 0, stream>>>(A);
        rglru_carry_kernel<<<(W + 63) / 64, 64, 0, stream>>>(A, chunks);
    }
    rglru_scan_kernel<1><<<grid, 256, 0, stream>>>(A);
    if (A.fin) rglru_states_kernel<<<dim3((W + 255) / 256, n_seqs), 256, 0, stream>>>(A);
    AGAVE_LAUNCH_CHECK("rglru_scan");
    return 0;
}
