// A gated linear recurrence per channel (the recurrent unit of Griffin's recurrent block) for gfx950.
//
//   r = sigmoid(A_r[b] u_b + b_r[b]),  g = sigmoid(A_i[b] u_b + b_i[b])      in each of `blocks` equal parts b of the channels
//   log a = -decay r        (decay = c softplus(lam), made once on the host)
//   S <- a S + sqrt(1 - a^2) g u          out = S gelu_tanh(y)
//
// rglru_gates: the two block-diagonal products and everything up to (a, sqrt(1 - a^2) g u), in 32-bit whatever the
// element type of the gate matrices.  A workgroup takes 32 tokens x 64 channels of a block; the inputs and both
// matrices' tiles pass through LDS in steps of 32 along the block.
// rglru_scan: S_t = a_t S_(t-1) + x_t along each sequence, over the step's rows in chunks: a chunk's effect on what
// comes in is (P, Q) with S_end = P S_in + Q (summarise), the chunks' carries follow one after another (carry), then
// every chunk runs again from its carry and writes the rows (apply).  A sequence's first row of the step starts from
// the sequence's state, its last row leaves the state.  Steps of few rows are one chunk and one launch.
#include "common_impl.h"
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

extern "C" int agave_rglru_gates(int w_dtype, const float* u, long ldu, const void* wr, const void* wi, const float* br,
                                 const float* bi, const float* decay, float* a_out, float* x_out, int N, int W, int blocks,
                                 hipStream_t stream) {
    AGAVE_CHECK(u && wr && wi && br && bi && decay && a_out && x_out, "rglru_gates: null buffer");
    AGAVE_CHECK(N >= 0 && W > 0 && blocks > 0 && W % blocks == 0 && ldu >= W, "rglru_gates: %d channels in %d blocks, row stride %ld", W, blocks, ldu);
    if (N == 0) return 0;
    const int bw = W / blocks;
    const dim3 grid((N + GT - 1) / GT, blocks, (bw + GO - 1) / GO);
    AGAVE_CHECK(grid.y <= 65535 && grid.z <= 65535, "rglru_gates: too many blocks");
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
template <int MODE>
__global__ __launch_bounds__(256) void rglru_scan_kernel(ScanArgs A) {
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch >= A.W) return;
    const int k = blockIdx.y;
    const int t0 = k * A.L, t1 = min(A.N, t0 + A.L);
    float P = 1.f, S = (MODE == 1 && k > 0) ? A.carry[(size_t)k * A.W + ch] : 0.f;
    for (int t = t0; t < t1; ++t) {
        const int b = A.tok_seq[t];
        const bool first = t == A.cu[b], last = t + 1 == A.cu[b + 1];
        if (first) {
            S = A.state[(size_t)A.slots[b] * A.W + ch];
            P = 0.f;
        }
        const float a = A.a[(size_t)t * A.W + ch];
        S = fmaf(a, S, A.x[(size_t)t * A.W + ch]);
        P *= a;
        if (MODE == 1) {
            const float v = S * gelu_tanh_f(A.y[(size_t)t * A.ldy + ch]);
            if (A.out_dtype == AGAVE_F32) ((float*)A.out)[(size_t)t * A.ldo + ch] = v;
            else ((bf16*)A.out)[(size_t)t * A.ldo + ch] = f32_to_bf16(v);
            if (last) {
                if (A.fin) A.fin[(size_t)b * A.W + ch] = S;
                else A.state[(size_t)A.slots[b] * A.W + ch] = S;
            }
        }
    }
    if (MODE == 0) {
        A.P[(size_t)k * A.W + ch] = P;
        A.Q[(size_t)k * A.W + ch] = S;
    }
}

// carry[k] = what enters chunk k: carry[k + 1] = P[k] carry[k] + Q[k] (chunk 0 always starts at a sequence's first row)
__global__ __launch_bounds__(256) void rglru_carry_kernel(ScanArgs A, int chunks) {
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch >= A.W) return;
    float S = 0.f;
    for (int k = 0; k + 1 < chunks; ++k) {
        S = fmaf(A.P[(size_t)k * A.W + ch], S, A.Q[(size_t)k * A.W + ch]);
        A.carry[(size_t)(k + 1) * A.W + ch] = S;
    }
}

__global__ __launch_bounds__(256) void rglru_states_kernel(ScanArgs A) {
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    if (ch < A.W) A.state[(size_t)A.slots[blockIdx.y] * A.W + ch] = A.fin[(size_t)blockIdx.y * A.W + ch];
}

extern "C" int agave_rglru_scan(const float* a, const float* x, const float* y, long ldy, void* out, int out_dtype, long ldo,
                                float* state, const int* tok_seq, const int* cu, const int* slots, float* scratch,
                                long scratch_floats, int N, int n_seqs, int W, int L, hipStream_t stream) {
    AGAVE_CHECK(a && x && y && out && state && tok_seq && cu && slots, "rglru_scan: null buffer");
    AGAVE_CHECK(N >= 0 && W > 0 && L > 0 && ldy >= W && ldo >= W, "rglru_scan: bad sizes N=%d W=%d L=%d", N, W, L);
    AGAVE_CHECK(out_dtype == AGAVE_F32 || out_dtype == AGAVE_BF16, "rglru_scan: unknown dtype %d", out_dtype);
    if (N == 0) return 0;
    const int chunks = (N + L - 1) / L;
    AGAVE_CHECK(chunks <= 65535, "rglru_scan: %d chunks of rows", chunks);
    ScanArgs A{a, x, y, ldy, out, out_dtype, ldo, state, tok_seq, cu, slots, nullptr, nullptr, nullptr, nullptr, N, W, L};
    const dim3 grid((W + 255) / 256, chunks);
    if (chunks > 1) {
        const long need = (3L * chunks + n_seqs) * W;
        AGAVE_CHECK(n_seqs > 0 && n_seqs <= 65535 && scratch && scratch_floats >= need, "rglru_scan: %d chunks and %d sequences need %ld floats of scratch", chunks, n_seqs, need);
        A.fin = scratch + 3 * (size_t)chunks * W;
        A.P = scratch;
        A.Q = scratch + (size_t)chunks * W;
        A.carry = scratch + 2 * (size_t)chunks * W;
        rglru_scan_kernel<0><<<grid, 256, 0, stream>>>(A);
        rglru_carry_kernel<<<(W + 255) / 256, 256, 0, stream>>>(A, chunks);
    }
    rglru_scan_kernel<1><<<grid, 256, 0, stream>>>(A);
    if (A.fin) rglru_states_kernel<<<dim3((W + 255) / 256, n_seqs), 256, 0, stream>>>(A);
    AGAVE_LAUNCH_CHECK("rglru_scan");
    return 0;
}
