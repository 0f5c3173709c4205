// Kernels of the attention whose keys and values come from one small latent row per position, for gfx950:
//
//   latent_prepare   the two latents of a token: the query latent divided by its root mean square times a weight
//                    (the rows the query product reads), and the key/value latent likewise with its last elements,
//                    which are not normed, rotated by the position: the row [c | r] that the cache holds;
//   heads_product    a small product per (token, head): y[t][h] = W[h] x[t][h], for the step that folds a head's key
//                    matrix into its query (so that scores are taken against the cached rows themselves) and for the
//                    step that makes a head's values from the attention's sum over latent rows; it can copy a
//                    head's trailing elements behind the product while rotating them, and multiply the result by
//                    the sigmoid of a gate.
//   latent_expand    for a prompt that starts at its first position, where every head's own keys are made from the
//                    latent rows instead (fewer multiplications than the folded form when rows are many): the
//                    rotated key part is put behind every head's unrotated keys, and the queries' trailing elements
//                    are rotated in place;
//   gate_rows        rows times the sigmoid of 32-bit logits, in place.
//
// Norm sums, angles, sines and the products' sums are 32-bit; T is the element type of the rows between products.
#include "common_impl.h"
#include "mfma.h"
#include <math.h>

// the pair (u, v) = (x[i], x[i + half]) at position p turns by the angle p * freq[i]
__device__ __forceinline__ void turn(float u, float v, float angle, float& uo, float& vo) {
    float s, c;
    sincosf(angle, &s, &c);
    uo = u * c - v * s;
    vo = v * c + u * s;
}

// grid (tokens, 2): y = 0 the query latent, y = 1 the key/value latent (absent where kv is null)
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(const float* __restrict__ qraw, long ldq, const float* __restrict__ qw,
                                                             T* __restrict__ cq, long ldcq, int q_rank,
                                                             const float* __restrict__ kvraw, long ldkv,
                                                             const float* __restrict__ kvw, T* __restrict__ krow, long ldkr,
                                                             int kv_rank, int rot_dim, const float* __restrict__ freq,
                                                             int rot_half, const int* __restrict__ tok_pos, float eps) {
    __shared__ float red[16];
    const int t = blockIdx.x, tid = threadIdx.x;
    const bool kv = blockIdx.y == 1;
    const float* x = kv ? kvraw + (size_t)t * ldkv : qraw + (size_t)t * ldq;
    const float* w = kv ? kvw : qw;
    T* out = kv ? krow + (size_t)t * ldkr : cq + (size_t)t * ldcq;
    const int n = kv ? kv_rank : q_rank;
    float ss = 0.f;
    for (int e = tid; e < n; e += 256) ss = fmaf(x[e], x[e], ss);
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (int e = tid; e < n; e += 256) st(out + e, x[e] * inv * w[e]);
    if (!kv) return;
    const float p = (float)tok_pos[t];
    const float* r = x + kv_rank;
    for (int e = tid; e < rot_dim; e += 256) {
        float y = r[e];
        if (e < rot_half) {
            float o2;
            turn(r[e], r[e + rot_half], p * freq[e], y, o2);
        } else if (e < 2 * rot_half) {
            float o1;
            turn(r[e - rot_half], r[e], p * freq[e - rot_half], o1, y);
        }
        st(out + kv_rank + e, y);
    }
}

extern "C" int agave_latent_prepare(int dtype, const float* qraw, long ldq, const float* qw, void* cq, long ldcq, int q_rank,
                                    const float* kvraw, long ldkv, const float* kvw, void* krow, long ldkr, int kv_rank,
                                    int rot_dim, const float* freq, int rot_half, const int* tok_pos, int n_tokens, float eps,
                                    hipStream_t stream) {
    AGAVE_CHECK(n_tokens >= 0 && q_rank > 0, "latent_prepare: bad sizes N=%d q_rank=%d", n_tokens, q_rank);
    AGAVE_CHECK(qraw && qw && cq && ldq >= q_rank && ldcq >= q_rank, "latent_prepare: bad query buffers");
    if (kvraw) {
        AGAVE_CHECK(kv_rank > 0 && rot_dim >= 0 && 2 * rot_half <= rot_dim, "latent_prepare: bad sizes kv_rank=%d rot_dim=%d rotated=%d",
                    kv_rank, rot_dim, 2 * rot_half);
        AGAVE_CHECK(kvw && krow && tok_pos && (freq || rot_half == 0) && ldkv >= kv_rank + rot_dim && ldkr >= kv_rank + rot_dim,
                    "latent_prepare: bad key/value buffers");
    }
    if (n_tokens == 0) return 0;
    const dim3 grid(n_tokens, kvraw ? 2 : 1);
    if (dtype == AGAVE_F32)
        latent_prepare_kernel<float><<<grid, 256, 0, stream>>>(qraw, ldq, qw, (float*)cq, ldcq, q_rank, kvraw, ldkv, kvw, (float*)krow,
                                                               ldkr, kv_rank, rot_dim, freq, rot_half, tok_pos, eps);
    else if (dtype == AGAVE_BF16)
        latent_prepare_kernel<bf16><<<grid, 256, 0, stream>>>(qraw, ldq, qw, (bf16*)cq, ldcq, q_rank, kvraw, ldkv, kvw, (bf16*)krow,
                                                              ldkr, kv_rank, rot_dim, freq, rot_half, tok_pos, eps);
    else
        AGAVE_CHECK(false, "latent_prepare: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("latent_prepare");
    return 0;
}

// ------------------------------------------------------------------ a product per (token, head)
//   y[t][h][c] = sum_k W[h][c][k] x[t][h * xs + k]        (c < n_out, k < K;  W is [heads][n_out][K])
//   y[t][h][n_out + e] = the head's elements x[t][h * xs + K + e], e < tail, the first 2 * rot_half of them rotated
//   y[t][h][c] *= sigmoid(gate[t][h * n_out + c])          (where a gate is given; it is 32-bit)
// y's head h starts at column h * ys.
struct HeadsProductArgs {
    const void* x; long ldx; int xs;
    const void* w;
    void* y; long ldy; int ys;
    const float* gate; long ldg;
    const float* freq; int rot_half; int tail;
    const int* tok_pos;
    int n_tokens, heads, n_out, K;
};

// The plain form: a workgroup per (token, head), the head's input in LDS, a wave per output column in turn with
// the lanes along K.  Any sizes, both element types.
template <typename T>
__global__ __launch_bounds__(256) void heads_product_plain_kernel(HeadsProductArgs A) {
    extern __shared__ float xh[];                       // [K + tail]
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const T* x = (const T*)A.x + (size_t)t * A.ldx + (size_t)h * A.xs;
    for (int k = tid; k < A.K + A.tail; k += 256) xh[k] = ld(x + k);
    __syncthreads();
    T* y = (T*)A.y + (size_t)t * A.ldy + (size_t)h * A.ys;
    const T* w = (const T*)A.w + (size_t)h * A.n_out * A.K;
    for (int c = wv; c < A.n_out; c += 4) {
        const T* wr = w + (size_t)c * A.K;
        float acc = 0.f;
        for (int k = lane; k < A.K; k += 64) acc = fmaf(ld(wr + k), xh[k], acc);
        acc = wave_sum(acc);
        if (lane == 0) {
            if (A.gate) acc *= 1.0f / (1.0f + expf(-A.gate[(size_t)t * A.ldg + (size_t)h * A.n_out + c]));
            st(y + c, acc);
        }
    }
    if (A.tail) {
        const float p = (float)A.tok_pos[t];
        const float* r = xh + A.K;
        for (int e = tid; e < A.tail; e += 256) {
            float o = r[e];
            if (e < A.rot_half) {
                float o2;
                turn(r[e], r[e + A.rot_half], p * A.freq[e], o, o2);
            } else if (e < 2 * A.rot_half) {
                float o1;
                turn(r[e - A.rot_half], r[e], p * A.freq[e - A.rot_half], o1, o);
            }
            st(y + A.n_out + e, o);
        }
    }
}

// The matrix cores' form (bfloat16; K a multiple of 8, aligned rows): a workgroup takes 64 tokens of one head and 64
// output columns (or, in a step of up to 16 tokens, those tokens and 256 columns); each of its four waves 16 tokens against 64 columns, both operands straight from memory in the
// order v_mfma_f32_16x16x32_bf16 reads them (a lane's eight neighbours along K are 16 bytes of a row).  The head's
// weights are small and stay in the caches; what the kernel moves is the rows.  The trailing elements are copied,
// rotated, by the workgroups of the first column block.
__global__ __launch_bounds__(256) void heads_product_mfma_kernel(HeadsProductArgs A) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int h = blockIdx.y;
    // up to 16 tokens (a decode step): the four waves take four blocks of columns of the same 16 rows
    const bool few = A.n_tokens <= 16;
    const int row0 = few ? 0 : blockIdx.x * 64 + wv * 16;
    const int col0 = few ? (blockIdx.z * 4 + wv) * 64 : blockIdx.z * 64;
    const int K = A.K, n_out = A.n_out;
    if (col0 >= n_out || row0 >= A.n_tokens) return;            // (no barrier below)
    const bf16* x = (const bf16*)A.x;
    const bf16* w = (const bf16*)A.w + (size_t)h * n_out * K;
    bf16* y = (bf16*)A.y;
    int trow = row0 + c;
    trow = trow < A.n_tokens ? trow : A.n_tokens - 1;
    const bf16* arow = x + (size_t)trow * A.ldx + (size_t)h * A.xs + 8 * g;
    const bf16* brow[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int col = col0 + 16 * j + c;
        col = col < n_out ? col : n_out - 1;
        brow[j] = w + (size_t)col * K + 8 * g;
    }
    f32x4_t acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    // four steps along K at a time: their loads leave together (without conditions, from inside the row; a lane past the
    // row's end reads its start and is emptied), so a product is a few round trips to memory and not one per step
    for (int k0 = 0; k0 < K; k0 += 128) {
        frag16 a[4], b[4][4];
        bool in[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            in[u] = k0 + 32 * u + 8 * g < K;
            const int at = in[u] ? k0 + 32 * u : -8 * g;
            a[u].u = *reinterpret_cast<const uint4*>(arow + at);
#pragma unroll
            for (int j = 0; j < 4; ++j) b[u][j].u = *reinterpret_cast<const uint4*>(brow[j] + at);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (!in[u]) a[u].u = make_uint4(0, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = mfma_16x16x32(a[u], b[u][j], acc[j]);
        }
    }
    // D[j]: the lane holds tokens row0 + 4 g + e4, column col0 + 16 j + c
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int col = col0 + 16 * j + c;
        if (col >= n_out) continue;
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
            const int t = row0 + 4 * g + e4;
            if (t >= A.n_tokens) continue;
            float v = acc[j][e4];
            if (A.gate) v *= 1.0f / (1.0f + expf(-A.gate[(size_t)t * A.ldg + (size_t)h * n_out + col]));
            y[(size_t)t * A.ldy + (size_t)h * A.ys + col] = f32_to_bf16(v);
        }
    }
    if (A.tail && col0 == 0) {
        for (int i = lane; i < 16 * A.tail; i += 64) {
            const int t = row0 + i / A.tail, e = i % A.tail;
            if (t >= A.n_tokens) continue;
            const bf16* r = x + (size_t)t * A.ldx + (size_t)h * A.xs + K;
            const float p = (float)A.tok_pos[t];
            float o = bf16_to_f32(r[e]);
            if (e < A.rot_half) {
                float o2;
                turn(o, bf16_to_f32(r[e + A.rot_half]), p * A.freq[e], o, o2);
            } else if (e < 2 * A.rot_half) {
                float o1;
                turn(bf16_to_f32(r[e - A.rot_half]), o, p * A.freq[e - A.rot_half], o1, o);
            }
            y[(size_t)t * A.ldy + (size_t)h * A.ys + n_out + e] = f32_to_bf16(o);
        }
    }
}

extern "C" int agave_heads_product(int dtype, const void* x, long ldx, int xs, const void* w, void* y, long ldy, int ys,
                                   const float* gate, long ldg, const float* freq, int rot_half, int tail, const int* tok_pos,
                                   int n_tokens, int heads, int n_out, int K, int plain, hipStream_t stream) {
    AGAVE_CHECK(n_tokens >= 0 && heads > 0 && n_out > 0 && K > 0 && tail >= 0, "heads_product: bad sizes N=%d heads=%d out=%d K=%d", n_tokens, heads, n_out, K);
    AGAVE_CHECK(x && w && y, "heads_product: null buffer");
    AGAVE_CHECK(xs >= K + tail && ldx >= (long)(heads - 1) * xs + K + tail, "heads_product: the input's rows are too short");
    AGAVE_CHECK(ys >= n_out + tail && ldy >= (long)(heads - 1) * ys + n_out + tail, "heads_product: the output's rows are too short");
    AGAVE_CHECK(!gate || ldg >= (long)heads * n_out, "heads_product: the gate's rows are too short");
    AGAVE_CHECK(2 * rot_half <= tail && (tail == 0 || (tok_pos && (freq || rot_half == 0))), "heads_product: %d rotated of %d trailing elements", 2 * rot_half, tail);
    AGAVE_CHECK(heads <= 65535 && (K + tail) * sizeof(float) <= 64 * 1024, "heads_product: too many heads or too long a head");
    if (n_tokens == 0) return 0;
    HeadsProductArgs A{x, ldx, xs, w, y, ldy, ys, gate, ldg, freq, rot_half, tail, tok_pos, n_tokens, heads, n_out, K};
    const bool mfma = !plain && dtype == AGAVE_BF16 && K % 8 == 0 && xs % 8 == 0 && ldx % 8 == 0 &&
                      ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0;
    if (mfma) {
        const dim3 grid = n_tokens <= 16 ? dim3(1, heads, (n_out + 255) / 256) : dim3((n_tokens + 63) / 64, heads, (n_out + 63) / 64);
        AGAVE_CHECK(grid.z <= 65535, "heads_product: too many columns");
        heads_product_mfma_kernel<<<grid, 256, 0, stream>>>(A);
    } else {
        const dim3 grid(n_tokens, heads);
        const size_t lds = (size_t)(K + tail) * sizeof(float);
        if (dtype == AGAVE_F32) heads_product_plain_kernel<float><<<grid, 256, lds, stream>>>(A);
        else if (dtype == AGAVE_BF16) heads_product_plain_kernel<bf16><<<grid, 256, lds, stream>>>(A);
        else AGAVE_CHECK(false, "heads_product: unknown dtype %d", dtype);
    }
    AGAVE_LAUNCH_CHECK("heads_product");
    return 0;
}


// ------------------------------------------------------------------ every head's key row from the latent's parts
//   kfull[t][h] = [ knope[t][h] (dim elements) | krow[t][kv_rank ..] (rot_dim elements, already rotated) ]
//   q[t][h][dim + e], e < rot_dim: the first 2 * rot_half of them rotated in pairs (e, e + rot_half), in place
// A workgroup per token.
template <typename T>
__global__ __launch_bounds__(256) void latent_expand_kernel(T* __restrict__ q, long ldq, const T* __restrict__ knope, long ldkn,
                                                            const T* __restrict__ krow, long ldkr, int kv_rank, T* __restrict__ kfull,
                                                            long ldkf, const float* __restrict__ freq, int rot_half,
                                                            const int* __restrict__ tok_pos, int heads, int dim, int rot_dim) {
    const int t = blockIdx.x, tid = threadIdx.x, qd = dim + rot_dim;
    const T* kn = knope + (size_t)t * ldkn;
    const T* r = krow + (size_t)t * ldkr + kv_rank;
    T* kf = kfull + (size_t)t * ldkf;
    for (int i = tid; i < heads * qd; i += 256) {
        const int h = i / qd, e = i % qd;
        kf[i] = e < dim ? kn[(size_t)h * dim + e] : r[e - dim];
    }
    const float p = (float)tok_pos[t];
    T* qr = q + (size_t)t * ldq;
    // (a thread takes a whole pair, so nothing is read after it was written)
    for (int i = tid; i < heads * rot_half; i += 256) {
        const int h = i / rot_half, e = i % rot_half;
        T* a = qr + (size_t)h * qd + dim + e;
        float u, v;
        turn(ld(a), ld(a + rot_half), p * freq[e], u, v);
        st(a, u);
        st(a + rot_half, v);
    }
}

extern "C" int agave_latent_expand(int dtype, void* q, long ldq, const void* knope, long ldkn, const void* krow, long ldkr,
                                   int kv_rank, void* kfull, long ldkf, const float* freq, int rot_half, const int* tok_pos,
                                   int n_tokens, int heads, int dim, int rot_dim, hipStream_t stream) {
    AGAVE_CHECK(n_tokens >= 0 && heads > 0 && dim > 0 && rot_dim >= 0 && kv_rank > 0 && 2 * rot_half <= rot_dim,
                "latent_expand: bad sizes N=%d heads=%d dim=%d rot_dim=%d rotated=%d", n_tokens, heads, dim, rot_dim, 2 * rot_half);
    AGAVE_CHECK(q && knope && krow && kfull && tok_pos && (freq || rot_half == 0), "latent_expand: null buffer");
    AGAVE_CHECK(ldq >= (long)heads * (dim + rot_dim) && ldkf >= (long)heads * (dim + rot_dim) && ldkn >= (long)heads * dim &&
                ldkr >= kv_rank + rot_dim, "latent_expand: a row stride is too small");
    if (n_tokens == 0) return 0;
    if (dtype == AGAVE_F32)
        latent_expand_kernel<float><<<n_tokens, 256, 0, stream>>>((float*)q, ldq, (const float*)knope, ldkn, (const float*)krow, ldkr,
                                                                  kv_rank, (float*)kfull, ldkf, freq, rot_half, tok_pos, heads, dim, rot_dim);
    else if (dtype == AGAVE_BF16)
        latent_expand_kernel<bf16><<<n_tokens, 256, 0, stream>>>((bf16*)q, ldq, (const bf16*)knope, ldkn, (const bf16*)krow, ldkr,
                                                                 kv_rank, (bf16*)kfull, ldkf, freq, rot_half, tok_pos, heads, dim, rot_dim);
    else
        AGAVE_CHECK(false, "latent_expand: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("latent_expand");
    return 0;
}

// ------------------------------------------------------------------ x *= sigmoid(gate), gate in 32-bit
template <typename T>
__global__ void gate_rows_kernel(T* __restrict__ x, long ldx, const float* __restrict__ gate, long ldg, long total, int cols) {
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
        const long r = idx / cols;
        const int c = (int)(idx % cols);
        T* at = x + r * ldx + c;
        st(at, ld(at) * (1.0f / (1.0f + expf(-gate[r * ldg + c]))));
    }
}

extern "C" int agave_gate_rows(int dtype, void* x, long ldx, const float* gate, long ldg, int rows, int cols, hipStream_t stream) {
    AGAVE_CHECK(rows >= 0 && cols > 0 && ldx >= cols && ldg >= cols && x && gate, "gate_rows: bad sizes rows=%d cols=%d", rows, cols);
    if (rows == 0) return 0;
    const long total = (long)rows * cols;
    long blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == AGAVE_F32) gate_rows_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)x, ldx, gate, ldg, total, cols);
    else if (dtype == AGAVE_BF16) gate_rows_kernel<bf16><<<(int)blocks, 256, 0, stream>>>((bf16*)x, ldx, gate, ldg, total, cols);
    else AGAVE_CHECK(false, "gate_rows: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("gate_rows");
    return 0;
}
