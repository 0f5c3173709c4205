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

// The same for 1 to 8 streams of a width that is a multiple of 4, with aligned rows: four neighbouring columns a thread
// (16-byte accesses), the number of streams known when the kernel is compiled (every load is written without a
// condition and all of a thread's loads leave before the first is used), and as many threads a token as the width
// has groups of four, so that a step of few tokens is one round of loads, two sums and one round of stores.
template <int S>
__global__ __launch_bounds__(1024) void streams_step_fast_kernel(StreamsArgs A) {
    extern __shared__ float u_row[];                 // [E]
    __shared__ float coef[S * S + 2 * S];
    __shared__ float red[16];
    const int E = A.E, E4 = E >> 2;
    const int t = A.rows ? A.rows[blockIdx.x] : (int)blockIdx.x;
    float* mixc = coef;
    float* wrc = coef + S * S;
    float* rdc = wrc + S;
    if (threadIdx.x < S * S) mixc[threadIdx.x] = A.y ? A.mix[threadIdx.x] : 0.f;
    if (threadIdx.x < S) {
        wrc[threadIdx.x] = A.y ? A.write[threadIdx.x] : 0.f;
        rdc[threadIdx.x] = A.read ? A.read[threadIdx.x] : 0.f;
    }
    __syncthreads();
    float4* hx = reinterpret_cast<float4*>(A.h + (size_t)t * S * E);
    float part = 0.f;
    for (int c = threadIdx.x; c < E4; c += blockDim.x) {
        float4 x[S];
#pragma unroll
        for (int s = 0; s < S; ++s) x[s] = hx[(size_t)s * E4 + c];
        float4 u = make_float4(0.f, 0.f, 0.f, 0.f);
        if (A.y) {
            float4 y = make_float4(0.f, 0.f, 0.f, 0.f);
            if (A.y_dtype == AGAVE_F32) {
                for (int sl = 0; sl < A.y_slices; ++sl) {
                    const float4 v = *reinterpret_cast<const float4*>((const float*)A.y + (size_t)sl * A.y_slice_stride + (size_t)t * A.ldy + 4 * c);
                    y.x += v.x; y.y += v.y; y.z += v.z; y.w += v.w;
                }
            } else {
                const uint2 v = *reinterpret_cast<const uint2*>((const bf16*)A.y + (size_t)t * A.ldy + 4 * c);
                y = make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                                __uint_as_float(v.y & 0xffff0000u));
            }
#pragma unroll
            for (int to = 0; to < S; ++to) {
                const float wv = wrc[to];
                float4 v = make_float4(wv * y.x, wv * y.y, wv * y.z, wv * y.w);
#pragma unroll
                for (int s = 0; s < S; ++s) {
                    const float m = mixc[s * S + to];
                    v.x = fmaf(m, x[s].x, v.x); v.y = fmaf(m, x[s].y, v.y); v.z = fmaf(m, x[s].z, v.z); v.w = fmaf(m, x[s].w, v.w);
                }
                if (A.store) hx[(size_t)to * E4 + c] = v;
                const float r = rdc[to];
                u.x = fmaf(r, v.x, u.x); u.y = fmaf(r, v.y, u.y); u.z = fmaf(r, v.z, u.z); u.w = fmaf(r, v.w, u.w);
            }
        } else {
#pragma unroll
            for (int s = 0; s < S; ++s) {
                const float r = rdc[s];
                u.x = fmaf(r, x[s].x, u.x); u.y = fmaf(r, x[s].y, u.y); u.z = fmaf(r, x[s].z, u.z); u.w = fmaf(r, x[s].w, u.w);
            }
        }
        reinterpret_cast<float4*>(u_row)[c] = u;
        part += (u.x + u.y) + (u.z + u.w);
    }
    if (!A.out) return;
    float mean = 0.f;
    if (A.norm_kind == 1) mean = block_sum(part, red) / (float)E;
    float sq = 0.f;
    for (int c = threadIdx.x; c < E4; c += blockDim.x) {             // (a thread reads back what it wrote itself)
        const float4 v = reinterpret_cast<const float4*>(u_row)[c];
        const float a = v.x - mean, b = v.y - mean, cc = v.z - mean, d = v.w - mean;
        sq += (a * a + b * b) + (cc * cc + d * d);
    }
    float inv = 1.f;
    if (A.norm_kind != 0) inv = 1.0f / sqrtf(block_sum(sq, red) / (float)E + A.eps);
    const size_t orow = (size_t)blockIdx.x * A.ldo;
    for (int c = threadIdx.x; c < E4; c += blockDim.x) {
        const float4 v = reinterpret_cast<const float4*>(u_row)[c];
        float o[4] = {(v.x - mean) * inv, (v.y - mean) * inv, (v.z - mean) * inv, (v.w - mean) * inv};
        if (A.norm_kind != 0) {
            const float4 w = reinterpret_cast<const float4*>(A.w)[c];
            const float4 b = A.b ? reinterpret_cast<const float4*>(A.b)[c] : make_float4(0.f, 0.f, 0.f, 0.f);
            o[0] = fmaf(o[0], w.x, b.x); o[1] = fmaf(o[1], w.y, b.y); o[2] = fmaf(o[2], w.z, b.z); o[3] = fmaf(o[3], w.w, b.w);
        }
        if (A.out_dtype == AGAVE_F32) {
            *reinterpret_cast<float4*>((float*)A.out + orow + 4 * c) = make_float4(o[0], o[1], o[2], o[3]);
        } else {
            uint2 pk;
            pk.x = f32x2_to_bf16x2(o[0], o[1]);
            pk.y = f32x2_to_bf16x2(o[2], o[3]);
            *reinterpret_cast<uint2*>((bf16*)A.out + orow + 4 * c) = pk;
        }
    }
}

template <int S>
static void launch_streams_fast(const StreamsArgs& A, int blocks, hipStream_t stream) {
    int threads = ((A.E / 4) + 63) / 64 * 64;
    threads = threads < 64 ? 64 : threads > 1024 ? 1024 : threads;
    streams_step_fast_kernel<S><<<blocks, threads, (size_t)A.E * sizeof(float), stream>>>(A);
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
    const bool aligned = E % 4 == 0 && ((uintptr_t)h % 16) == 0 &&
                         (!y || (ldy % 4 == 0 && y_slice_stride % 4 == 0 && ((uintptr_t)y % 16) == 0)) &&
                         (!out || (ldo % 4 == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)w % 16) == 0 && ((uintptr_t)b % 16) == 0));
    if (aligned && S <= 8) {
        switch (S) {
            case 1: launch_streams_fast<1>(A, blocks, stream); break;
            case 2: launch_streams_fast<2>(A, blocks, stream); break;
            case 3: launch_streams_fast<3>(A, blocks, stream); break;
            case 4: launch_streams_fast<4>(A, blocks, stream); break;
            case 5: launch_streams_fast<5>(A, blocks, stream); break;
            case 6: launch_streams_fast<6>(A, blocks, stream); break;
            case 7: launch_streams_fast<7>(A, blocks, stream); break;
            default: launch_streams_fast<8>(A, blocks, stream); break;
        }
    } else {
        streams_step_kernel<<<blocks, 256, (size_t)E * sizeof(float), stream>>>(A);
    }
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
