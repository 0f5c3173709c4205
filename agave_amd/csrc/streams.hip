// Several residual streams per token (hyper-connections) for gfx950.
//
// The residual of a token is S rows x_1 .. x_S of E floats, stored [token][stream][E] in 32-bit.  A sublayer reads
//   u = sum_s read[s] x_s
// and its result y comes back as
//   x_t <- sum_s mix[s][t] x_s + write[t] y          (all t at once, from the old rows)
// One kernel does the write of the sublayer that just ran and the read (with the norm in front of the next
// sublayer) of the one that runs next, so the streams are read and written once per sublayer:
//   streams_step:  [x <- mix^T x + write y]  then  [out = norm(sum_s read[s] x_s)]
// either half may be missing.  With `rows` the kernel visits only the chosen tokens and stores no streams (the
// model's end: the streams' sum of the wanted rows through the final norm).  The norm is a layer norm (weight
// and optional bias), an RMS norm (weight) or none; sums, mean and variance are 32-bit, the variance is the
// mean of the squared deviations from the mean (a second pass over the row, which waits in LDS).
#include "common_impl.h"
#include <math.h>

#define STREAMS_MAX 16
#define STREAMS_MAX_WIDTH 15360

struct StreamsArgs {
    float* h; int S; int E;
    const void* y; int y_dtype; long ldy; int y_slices; long y_slice_stride;     // null: nothing to write
    const float* mix; const float* write;            // [S][S] (from, to), [S]
    const float* read;                               // [S]; null: nothing to read
    int norm_kind;                                   // 0 none, 1 layer norm, 2 RMS norm
    const float* w; const float* b; float eps;
    void* out; int out_dtype; long ldo;
    const int* rows; int store;
};

__global__ __launch_bounds__(256) void streams_step_kernel(StreamsArgs A) {
    extern __shared__ float u_row[];                 // [E]
    __shared__ float coef[STREAMS_MAX * STREAMS_MAX + 2 * STREAMS_MAX];
    __shared__ float red[16];
    const int S = A.S, E = A.E;
    const int t = A.rows ? A.rows[blockIdx.x] : (int)blockIdx.x;
    float* mixc = coef;
    float* wrc = coef + STREAMS_MAX * STREAMS_MAX;
    float* rdc = wrc + STREAMS_MAX;
    for (int i = threadIdx.x; i < S * S; i += blockDim.x) mixc[i] = A.y ? A.mix[i] : ((i / S) == (i % S) ? 1.f : 0.f);
    for (int i = threadIdx.x; i < S; i += blockDim.x) {
        wrc[i] = A.y ? A.write[i] : 0.f;
        rdc[i] = A.read ? A.read[i] : 0.f;
    }
    __syncthreads();
    float* hx = A.h + (size_t)t * S * E;
    float part = 0.f;
    for (int c = threadIdx.x; c < E; c += blockDim.x) {
        float x[STREAMS_MAX];
#pragma unroll
        for (int s = 0; s < STREAMS_MAX; ++s) x[s] = s < S ? hx[(size_t)s * E + c] : 0.f;
        float u = 0.f;
        if (A.y) {
            float y = 0.f;
            for (int sl = 0; sl < A.y_slices; ++sl) {
                const size_t at = (size_t)sl * A.y_slice_stride + (size_t)t * A.ldy + c;
                y += A.y_dtype == AGAVE_F32 ? ((const float*)A.y)[at] : bf16_to_f32(((const bf16*)A.y)[at]);
            }
#pragma unroll
            for (int to = 0; to < STREAMS_MAX; ++to) {
                if (to < S) {
                    float v = wrc[to] * y;
#pragma unroll
                    for (int s = 0; s < STREAMS_MAX; ++s)
                        if (s < S) v = fmaf(mixc[s * S + to], x[s], v);
                    if (A.store) hx[(size_t)to * E + c] = v;
                    u = fmaf(rdc[to], v, u);
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < STREAMS_MAX; ++s)
                if (s < S) u = fmaf(rdc[s], x[s], u);
        }
        u_row[c] = u;
        part += u;
    }
    if (!A.out) return;
    float mean = 0.f;
    if (A.norm_kind == 1) mean = block_sum(part, red) / (float)E;
    float sq = 0.f;
    for (int c = threadIdx.x; c < E; c += blockDim.x) {
        const float d = u_row[c] - mean;
        sq = fmaf(d, d, sq);
    }
    float inv = 1.f;
    if (A.norm_kind != 0) inv = 1.0f / sqrtf(block_sum(sq, red) / (float)E + A.eps);
    const size_t orow = (size_t)blockIdx.x * A.ldo;
    for (int c = threadIdx.x; c < E; c += blockDim.x) {
        float v = (u_row[c] - mean) * inv;
        if (A.norm_kind != 0) v = v * A.w[c] + (A.b ? A.b[c] : 0.f);
        if (A.out_dtype == AGAVE_F32) ((float*)A.out)[orow + c] = v;
        else ((bf16*)A.out)[orow + c] = f32_to_bf16(v);
    }
}

extern "C" int agave_streams_step(float* h, int N, int S, int E, const void* y, int y_dtype, long ldy, int y_slices,
                                  long y_slice_stride, const float* mix, const float* write, const float* read, int norm_kind,
                                  const float* w, const float* b, float eps, void* out, int out_dtype, long ldo,
                                  const int* rows, int n_rows, hipStream_t stream) {
    AGAVE_CHECK(h && N >= 0 && S >= 1 && S <= STREAMS_MAX && E >= 1 && E <= STREAMS_MAX_WIDTH,
                "streams_step: %d streams of %d elements (1 to %d streams, up to %d elements)", S, E, STREAMS_MAX, STREAMS_MAX_WIDTH);
    AGAVE_CHECK(!y || (mix && write && y_slices >= 1 && ldy >= E && (y_dtype == AGAVE_F32 || y_dtype == AGAVE_BF16)),
                "streams_step: a result to write needs its coefficients and rows of the width");
    AGAVE_CHECK(!out || (read && ldo >= E && (out_dtype == AGAVE_F32 || out_dtype == AGAVE_BF16)),
                "streams_step: rows to hand on need the coefficients they are read with");
    AGAVE_CHECK(norm_kind >= 0 && norm_kind <= 2 && (norm_kind == 0 || w), "streams_step: norm %d without its weight", norm_kind);
    AGAVE_CHECK(!rows || out, "streams_step: chosen rows are for handing rows on");
    const int blocks = rows ? n_rows : N;
    if (blocks <= 0 || (!y && !out)) return 0;
    StreamsArgs A{h, S, E, y, y_dtype, ldy, y_slices, y_slice_stride, mix, write, read, norm_kind, w, b, eps,
                  out, out_dtype, ldo, rows, rows ? 0 : 1};
    streams_step_kernel<<<blocks, 256, (size_t)E * sizeof(float), stream>>>(A);
    AGAVE_LAUNCH_CHECK("streams_step");
    return 0;
}

// Every stream of a token starts as the token's row: h[t][s][:] = x[t][:].
__global__ void streams_fill_kernel(const float* __restrict__ x, float* __restrict__ h, int S, int E) {
    const int t = blockIdx.x;
    for (int c = threadIdx.x; c < E; c += blockDim.x) {
        const float v = x[(size_t)t * E + c];
        for (int s = 0; s < S; ++s) h[((size_t)t * S + s) * E + c] = v;
    }
}

extern "C" int agave_streams_fill(const float* x, float* h, int N, int S, int E, hipStream_t stream) {
    AGAVE_CHECK(x && h && N >= 0 && S >= 1 && E >= 1, "streams_fill: bad sizes");
    if (N == 0) return 0;
    streams_fill_kernel<<<N, 256, 0, stream>>>(x, h, S, E);
    AGAVE_LAUNCH_CHECK("streams_fill");
    return 0;
}
