// Softmax attention with a bias on the scores that depends on the distance between query and
// key, over cache pages stored row by row, for gfx950.  What the callers may combine:
//   * keys and values of different sizes, grouped query heads;
//   * a window (a query at position p sees keys p-W+1 .. p) and first positions that stay
//     visible whatever the window (keys j < keep_first), at their true distances;
//   * the bias: none; a slope per head, score -= slope_h * (p - j); or a table per head over
//     distances, score += table[h][min(p - j, len - 1)] (the host folds any bucketing of
//     distances into the table);
//   * chunks: a query sees only keys of its own chunk of C positions (j / C == p / C), chunks counted from the
//     sequence's first position; a cap on the scaled scores, cap * tanh(scale q.k / cap), before the bias;
//   * a sink per head: exp(sink_h) is added to the softmax's denominator, with no key or value;
//   * a gate on the output rows: out *= sigmoid(gate), element by element.
// Scores, bias, softmax and the sums over values are 32-bit in every element type.
//
// Cache pages: K [page][kv head][64 rows][hd]; V transposed [page][kv head][vd][64 rows]; or both in the order the
// matrix-core kernel reads its operands (below), which is how a bfloat16 cache holds them where the sizes allow.
// Position j of sequence b lies in row j % 64 of the page in column col(j / 64) of table[b]:
//   col(i) = i < head ? i : head + i - base[b]        (base[b] >= head)
// so the first `head` columns are the pages that hold the kept first positions, and the
// columns after them run from the oldest page the window reaches (base[b]) to the newest.
//
// Kernels: rows into the cache; a plain kernel (a workgroup per token and head, any sizes, both
// element types, either page order); a matrix-core kernel for prompts and for decode steps
// (bfloat16, pages in operand order, keys in steps of 8 and values in steps of 16 up to 256).
#include "common_impl.h"
#include "mfma.h"
#include <math.h>

__device__ __forceinline__ int page_col(int pi, int pbase, int head) { return pi < head ? pi : head + pi - pbase; }

// Pages in operand order (bfloat16, for the matrix-core kernel): a (page, kv head) block of keys is
// [4 key blocks][ksl = ceil(hd / 32) steps][64 lanes][8], lane c + 16 g of (kb, ks) holding elements
// 32 ks + 8 g .. + 8 of key key_of(kb, c) (see the kernel); a block of values is [vd / 16][2][64][8], lane
// c + 16 g of (nb, h) holding keys 32 h + 8 g .. + 8 of value column 16 nb + c.  A wave reads an operand
// of either with one load of a kilobyte in a row.  Where the head size is no multiple of 32 the last
// step's upper lanes stay zero (pages start out zeroed and nothing is ever written there).
__device__ __forceinline__ size_t k_operand_at(int r, int d, int ksl) {
    const int h = r >> 5, g4 = (r & 31) >> 3, sub = r & 7;
    const int kb = 2 * h + (sub >> 2), i = 4 * g4 + (sub & 3);
    return ((size_t)(kb * ksl + (d >> 5)) * 64 + i + 16 * ((d & 31) >> 3)) * 8 + (d & 7);
}
__device__ __forceinline__ size_t v_operand_at(int d, int r) {
    return ((size_t)((d >> 4) * 2 + (r >> 5)) * 64 + (d & 15) + 16 * ((r & 31) >> 3)) * 8 + (r & 7);
}

// ------------------------------------------------------------------ k and v rows into their pages
template <typename T>
__global__ void kv_append_rows_kernel(const T* __restrict__ k, long ldk, const T* __restrict__ v, long ldv,
                                      T* __restrict__ k_pages, T* __restrict__ v_pages, const int* __restrict__ table,
                                      int width, const int* __restrict__ base, int head, int n_pages,
                                      const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, int nkv, int hd,
                                      int vd, int packed) {
    const int t = blockIdx.x;
    const int b = tok_seq[t], p = tok_pos[t];
    const int col = page_col(p / AGAVE_PAGE, base[b], head);
    if (col < 0 || col >= width) return;
    const long pg = table[(size_t)b * width + col];
    if (pg < 0 || pg >= n_pages) return;
    const int row = p % AGAVE_PAGE;
    const int ksl = (hd + 31) / 32;
    const size_t kblock = packed ? (size_t)AGAVE_PAGE * ksl * 32 : (size_t)AGAVE_PAGE * hd;
    for (int i = threadIdx.x; i < nkv * hd; i += blockDim.x) {
        const int g = i / hd, d = i % hd;
        k_pages[((size_t)pg * nkv + g) * kblock + (packed ? k_operand_at(row, d, ksl) : (size_t)row * hd + d)] = k[(size_t)t * ldk + i];
    }
    for (int i = threadIdx.x; i < nkv * vd; i += blockDim.x) {
        const int g = i / vd, d = i % vd;
        v_pages[((size_t)pg * nkv + g) * vd * AGAVE_PAGE + (packed ? v_operand_at(d, row) : (size_t)d * AGAVE_PAGE + row)] =
            v[(size_t)t * ldv + i];
    }
}

extern "C" int agave_kv_append_rows(int dtype, const void* k, long ldk, const void* v, long ldv, void* k_pages,
                                    void* v_pages, const int* table, int width, const int* base, int head, int n_pages,
                                    const int* tok_seq, const int* tok_pos, int N, int nkv, int hd, int vd, int packed,
                                    hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && nkv > 0 && hd > 0 && vd > 0, "kv_append_rows: bad sizes N=%d nkv=%d hd=%d vd=%d", N, nkv, hd, vd);
    AGAVE_CHECK(k && v && k_pages && v_pages && table && base && tok_seq && tok_pos && width > 0 && n_pages > 0,
                "kv_append_rows: null buffer or empty table");
    AGAVE_CHECK(ldk >= (long)nkv * hd && ldv >= (long)nkv * vd, "kv_append_rows: a row stride is too small");
    AGAVE_CHECK(head >= 0, "kv_append_rows: negative count of kept pages");
    AGAVE_CHECK(!packed || (dtype == AGAVE_BF16 && hd % 8 == 0 && vd % 16 == 0), "kv_append_rows: pages in operand order hold bfloat16, keys in steps of 8 and values in steps of 16");
    if (N == 0) return 0;
    if (dtype == AGAVE_F32)
        kv_append_rows_kernel<float><<<N, 128, 0, stream>>>((const float*)k, ldk, (const float*)v, ldv, (float*)k_pages,
                                                            (float*)v_pages, table, width, base, head, n_pages, tok_seq,
                                                            tok_pos, nkv, hd, vd, 0);
    else if (dtype == AGAVE_BF16)
        kv_append_rows_kernel<bf16><<<N, 128, 0, stream>>>((const bf16*)k, ldk, (const bf16*)v, ldv, (bf16*)k_pages,
                                                           (bf16*)v_pages, table, width, base, head, n_pages, tok_seq,
                                                           tok_pos, nkv, hd, vd, packed);
    else
        AGAVE_CHECK(false, "kv_append_rows: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("kv_append_rows");
    return 0;
}

// ------------------------------------------------------------------ q and k rows before they meet
// 32-bit rows of a step's q, k and v (the projections' results, side by side or apart) become the rows the attention
// reads and the cache holds: a bias per element is added where the mixer has biases; q and k are divided by the
// root mean square of their whole row (all heads side by side) and multiplied by a weight per element where the mixer
// has such a norm; the first 2 * half elements of every head are rotated, pair (e, e + half) by the angle
// pos * freq[e], sine and cosine times `magnitude`; v is only converted.  k and v go straight into their places in
// the cache pages (either order) where pages are given, else into rows.
// The angle is made in double from double frequencies and reduced to [-pi/4, pi/4] there; its sine and cosine are
// 32-bit (a token's once, for all its heads); sums of squares and the rotation are 32-bit.  A workgroup per token.
struct RowsArgs {
    const float* q; long ldq; const float* k; long ldk; const float* v; long ldv;
    const float* q_b; const float* k_b; const float* v_b;
    void* q_out; long ldqo; void* k_out; long ldko; void* v_out; long ldvo;
    const float* q_w; const float* k_w; float eps_q, eps_k;
    const double* freq; int half; float magnitude;
    const int* tok_pos; const int* tok_seq;
    void* k_pages; void* v_pages; const int* table; int width; const int* base; int head; int n_pages; int packed;
    int nh, nkv, hd, vd;
};

template <typename T>
__global__ __launch_bounds__(1024) void row_norm_rope_kernel(RowsArgs A) {
    __shared__ float cs[2][256];
    __shared__ float red[2][16];
    const int t = blockIdx.x;
    const int pos = A.tok_pos[t];
    const int half = A.half, hd = A.hd;
    const bool has_k = A.k != nullptr;
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        // the angle in double, less the nearest multiple of pi/2 (in double too); what is left lies in [-pi/4, pi/4],
        // where sine and cosine are short 32-bit polynomials (errors of a few 1e-8); the quadrant swaps and negates
        const double ang = (double)pos * A.freq[i];
        const double q = rint(ang * 0.63661977236758134308);
        const float r = (float)(ang - q * 1.57079632679489661923), r2 = r * r;
        const float sp = fmaf(r * r2, fmaf(r2, fmaf(r2, -1.9515295891e-4f, 8.3321608736e-3f), -1.6666654611e-1f), r);
        const float cp = fmaf(r2 * r2, fmaf(r2, fmaf(r2, 2.443315711809948e-5f, -1.388731625493765e-3f), 4.166664568298827e-2f),
                              fmaf(r2, -0.5f, 1.0f));
        const int quad = (int)((long long)q & 3);
        const float sn = (quad & 1) ? cp : sp, c = (quad & 1) ? sp : cp;
        cs[0][i] = ((quad == 1 || quad == 2) ? -c : c) * A.magnitude;
        cs[1][i] = ((quad & 2) ? -sn : sn) * A.magnitude;
    }
    // where this token's key and value rows live
    long pg = -1;
    int prow = 0;
    if (A.k_pages && has_k) {
        const int sb = A.tok_seq[t];
        const int col = page_col(pos / AGAVE_PAGE, A.base[sb], A.head);
        if (col >= 0 && col < A.width) pg = A.table[(size_t)sb * A.width + col];
        if (pg >= A.n_pages) pg = -1;
        prow = pos % AGAVE_PAGE;
    }
    const int ksl = (hd + 31) / 32;
    const size_t kblock = A.packed ? (size_t)AGAVE_PAGE * ksl * 32 : (size_t)AGAVE_PAGE * hd;
    const float* xq = A.q + (size_t)t * A.ldq;
    const float* xk = has_k ? A.k + (size_t)t * A.ldk : nullptr;
    const int nq = A.nh * hd, nk = A.nkv * hd;
    // both rows' sums of squares in one pass and one meeting of the workgroup (which also completes the table)
    float sq = 0.f, sk = 0.f;
    if (A.q_w)
        for (int i = threadIdx.x; i < nq; i += blockDim.x) {
            const float v = xq[i] + (A.q_b ? A.q_b[i] : 0.f);
            sq = fmaf(v, v, sq);
        }
    if (A.k_w && has_k)
        for (int i = threadIdx.x; i < nk; i += blockDim.x) {
            const float v = xk[i] + (A.k_b ? A.k_b[i] : 0.f);
            sk = fmaf(v, v, sk);
        }
    sq = wave_sum(sq);
    sk = wave_sum(sk);
    if ((threadIdx.x & 63) == 0) {
        red[0][threadIdx.x >> 6] = sq;
        red[1][threadIdx.x >> 6] = sk;
    }
    __syncthreads();
    float tq = 0.f, tk = 0.f;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) {
        tq += red[0][i];
        tk += red[1][i];
    }
    const float inv_q = A.q_w ? 1.0f / sqrtf(tq / (float)nq + A.eps_q) : 1.f;
    const float inv_k = (A.k_w && has_k) ? 1.0f / sqrtf(tk / (float)nk + A.eps_k) : 1.f;
    for (int side = 0; side < 2; ++side) {
        const float* x = side == 0 ? xq : xk;
        if (!x) continue;                                   // (the whole workgroup: a run that appends nothing has no k)
        const float* bias = side == 0 ? A.q_b : A.k_b;
        const float* w = side == 0 ? A.q_w : A.k_w;
        const int heads = side == 0 ? A.nh : A.nkv;
        const float inv = side == 0 ? inv_q : inv_k;
        const bool to_pages = side == 1 && A.k_pages;
        T* y = side == 0 ? (T*)A.q_out + (size_t)t * A.ldqo : (to_pages ? nullptr : (T*)A.k_out + (size_t)t * A.ldko);
        auto put = [&](int i, float v) {
            if (!to_pages) {
                st(y + i, v);
            } else if (pg >= 0) {
                const int g = i / hd, d = i % hd;
                st((T*)A.k_pages + ((size_t)pg * A.nkv + g) * kblock + (A.packed ? k_operand_at(prow, d, ksl) : (size_t)prow * hd + d), v);
            }
        };
        // (whether there are biases and weights is known outside the loops, so that no load stands under a condition
        // and a thread's loads of a pair leave together)
        auto rows = [&](auto has_b, auto has_w) {
            constexpr bool HB = decltype(has_b)::value != 0, HW = decltype(has_w)::value != 0;
            for (int idx = threadIdx.x; idx < heads * half; idx += blockDim.x) {           // the rotated pairs
                const int e = idx % half, i = (idx / half) * hd + e;
                float a = x[i], b = x[i + half];
                if (HB) {
                    a += bias[i];
                    b += bias[i + half];
                }
                a *= inv;
                b *= inv;
                if (HW) {
                    a *= w[i];
                    b *= w[i + half];
                }
                const float c = cs[0][e], sn = cs[1][e];
                put(i, a * c - b * sn);
                put(i + half, b * c + a * sn);
            }
            const int rest = hd - 2 * half;
            for (int idx = threadIdx.x; idx < heads * rest; idx += blockDim.x) {           // what is not rotated
                const int i = (idx / rest) * hd + 2 * half + idx % rest;
                float a = x[i];
                if (HB) a += bias[i];
                a *= inv;
                if (HW) a *= w[i];
                put(i, a);
            }
        };
        if (bias) {
            if (w) rows(IntC<1>{}, IntC<1>{}); else rows(IntC<1>{}, IntC<0>{});
        } else {
            if (w) rows(IntC<0>{}, IntC<1>{}); else rows(IntC<0>{}, IntC<0>{});
        }
    }
    if (has_k && A.v) {
        const int vd = A.vd;
        for (int i = threadIdx.x; i < A.nkv * vd; i += blockDim.x) {
            const float v = A.v[(size_t)t * A.ldv + i] + (A.v_b ? A.v_b[i] : 0.f);
            if (!A.v_pages) {
                st((T*)A.v_out + (size_t)t * A.ldvo + i, v);
            } else if (pg >= 0) {
                const int g = i / vd, d = i % vd;
                st((T*)A.v_pages + ((size_t)pg * A.nkv + g) * vd * AGAVE_PAGE + (A.packed ? v_operand_at(d, prow) : (size_t)d * AGAVE_PAGE + prow), v);
            }
        }
    }
}

extern "C" int agave_row_norm_rope(int dtype, const float* q, long ldq, const float* k, long ldk, const float* v, long ldv,
                                   const float* q_b, const float* k_b, const float* v_b,
                                   void* q_out, long ldqo, void* k_out, long ldko, void* v_out, long ldvo, const float* q_w,
                                   const float* k_w, float eps_q, float eps_k, const double* freq, int half, float magnitude,
                                   const int* tok_pos, const int* tok_seq, void* k_pages, void* v_pages, const int* table,
                                   int width, const int* base, int head, int n_pages, int packed,
                                   int N, int nh, int nkv, int hd, int vd, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && nh > 0 && nkv > 0 && hd > 0 && vd > 0, "row_norm_rope: bad sizes");
    AGAVE_CHECK(q && q_out && tok_pos && ldq >= (long)nh * hd && ldqo >= (long)nh * hd, "row_norm_rope: q rows missing or too short");
    AGAVE_CHECK(!k || (v && ldk >= (long)nkv * hd && ldv >= (long)nkv * vd), "row_norm_rope: k and v rows missing or too short");
    AGAVE_CHECK(!k || k_pages || (k_out && v_out && ldko >= (long)nkv * hd && ldvo >= (long)nkv * vd),
                "row_norm_rope: no place for the k and v rows");
    AGAVE_CHECK(!k_pages || (v_pages && table && base && tok_seq && width > 0 && n_pages > 0 && head >= 0),
                "row_norm_rope: cache pages without their table");
    AGAVE_CHECK(!packed || (dtype == AGAVE_BF16 && hd % 8 == 0 && vd % 16 == 0), "row_norm_rope: pages in operand order hold bfloat16, keys in steps of 8 and values in steps of 16");
    AGAVE_CHECK(half >= 0 && half <= 256 && 2 * half <= hd && (half == 0 || freq), "row_norm_rope: %d rotated pairs in a head of %d (at most 256, with their frequencies)", half, hd);
    if (N == 0) return 0;
    RowsArgs A{q, ldq, k, ldk, k ? v : nullptr, ldv, q_b, k_b, v_b, q_out, ldqo, k_out, ldko, v_out, ldvo, q_w, k_w, eps_q, eps_k,
               freq, half, magnitude, tok_pos, tok_seq, k ? k_pages : nullptr, k ? v_pages : nullptr, table, width, base, head,
               n_pages, packed, nh, nkv, hd, vd};
    // (few tokens: sixteen waves a token, so that a thread has two or three elements and the waves hide each other's waits)
    const int threads = N <= 64 ? 1024 : 256;
    if (dtype == AGAVE_F32) row_norm_rope_kernel<float><<<N, threads, 0, stream>>>(A);
    else if (dtype == AGAVE_BF16) row_norm_rope_kernel<bf16><<<N, threads, 0, stream>>>(A);
    else AGAVE_CHECK(false, "row_norm_rope: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("row_norm_rope");
    return 0;
}

// ------------------------------------------------------------------ what the attention kernels share
struct BiasedArgs {
    const void* q; long ldq;
    void* out; long ldo;
    const void* gate; long ldg;          // null: no gate
    const void* k_pages; const void* v_pages;
    const int* table; int width; const int* base; int head; int n_pages;
    const int* tok_seq; const int* tok_pos;
    int nh, nkv, hd, vd;
    float scale;
    int window;                          // 0: all earlier keys
    int keep_first;                      // keys j < keep_first stay visible
    int bias_mode;                       // 0 none, 1 slopes, 2 table over distances
    const float* bias; int bias_len;     // slopes [nh], or table [nh][bias_len]
    const float* sink;                   // [nh] or null
    int packed;                          // the pages are in operand order
    int chunk;                           // 0: none; C: only keys of the query's own chunk of C positions
    float softcap;                       // 0: none; cap: score <- cap * tanh(score / cap), before the bias
};

__device__ __forceinline__ float score_bias(const BiasedArgs& A, int h, int dist) {
    if (A.bias_mode == 1) return -A.bias[h] * (float)dist;
    if (A.bias_mode == 2) return A.bias[(size_t)h * A.bias_len + (dist < A.bias_len ? dist : A.bias_len - 1)];
    return 0.f;
}

// ------------------------------------------------------------------ plain kernel
#define BCHUNK 256           // keys per pass = 4 pages
#define BACC 4               // value size <= 1024

template <typename T>
__global__ __launch_bounds__(256) void attn_biased_plain_kernel(BiasedArgs A) {
    __shared__ float qs[1024];
    __shared__ float sc[BCHUNK];
    __shared__ long page_of[BCHUNK / AGAVE_PAGE];
    __shared__ float red[16];

    const int tid = threadIdx.x;
    const int nh = A.nh, nkv = A.nkv, hd = A.hd, vd = A.vd;
    const int t = blockIdx.x / nh, h = blockIdx.x % nh;
    const int kvh = h / (nh / nkv);
    const int b = A.tok_seq[t];
    const int p = A.tok_pos[t];
    int lo = A.window > 0 ? (p - A.window + 1 > 0 ? p - A.window + 1 : 0) : 0;
    if (A.chunk > 0) lo = max(lo, (p / A.chunk) * A.chunk);
    const int kept_end = A.keep_first < lo ? A.keep_first : lo;     // keys [0, kept_end) lie before the window
    const int pbase = A.base[b];
    const T* q = (const T*)A.q;
    const T* k_pages = (const T*)A.k_pages;
    const T* v_pages = (const T*)A.v_pages;

    for (int d = tid; d < hd; d += blockDim.x) qs[d] = ld(q + (size_t)t * A.ldq + (size_t)h * hd + d);
    __syncthreads();

    // the sink starts the running maximum and sum: it is one more term of the denominator
    float m = -INFINITY, l = 0.f;
    if (A.sink) {
        m = A.sink[h];
        l = 1.f;
    }
    float acc[BACC];
#pragma unroll
    for (int a = 0; a < BACC; ++a) acc[a] = 0.f;

    // two stretches of keys: the kept first positions that the window has left behind, then the window
    for (int part = 0; part < 2; ++part) {
        const int j_lo = part == 0 ? 0 : lo;
        const int j_hi = part == 0 ? kept_end - 1 : p;              // inclusive
        if (j_hi < j_lo) continue;
        for (int c0 = (j_lo / AGAVE_PAGE) * AGAVE_PAGE; c0 <= j_hi; c0 += BCHUNK) {
            if (tid < BCHUNK / AGAVE_PAGE) {
                const int first = c0 + tid * AGAVE_PAGE;
                long pg = -1;
                const int col = page_col(first / AGAVE_PAGE, pbase, A.head);
                if (first <= j_hi && col >= 0 && col < A.width) pg = A.table[(size_t)b * A.width + col];
                if (pg >= A.n_pages) pg = -1;
                page_of[tid] = pg;
            }
            __syncthreads();
            const int j = c0 + tid;
            const long pg = page_of[tid / AGAVE_PAGE];
            const bool valid = j >= j_lo && j <= j_hi && pg >= 0;
            float s = -INFINITY;
            if (valid) {
                float dot = 0.f;
                if (A.packed) {
                    const int ksl = (hd + 31) / 32;
                    const T* kblk = k_pages + ((size_t)pg * nkv + kvh) * AGAVE_PAGE * ksl * 32;
                    for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], ld(kblk + k_operand_at(j % AGAVE_PAGE, d, ksl)), dot);
                } else {
                    const T* kr = k_pages + (((size_t)pg * nkv + kvh) * AGAVE_PAGE + (j % AGAVE_PAGE)) * hd;
                    for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], ld(kr + d), dot);
                }
                s = dot * A.scale;
                if (A.softcap > 0.f) s = A.softcap * tanhf(s / A.softcap);
                s += score_bias(A, h, p - j);
            }
            const float cmax = block_max(s, red);
            const float m_new = fmaxf(m, cmax);
            const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
            const float pr = valid ? expf(s - m_new) : 0.f;
            sc[tid] = pr;
            const float csum = block_sum(pr, red);      // has barriers: sc[] is visible afterwards
            l = l * alpha + csum;
            m = m_new;
#pragma unroll
            for (int a = 0; a < BACC; ++a) {
                const int d = tid + a * 256;
                if (d < vd) {
                    float sum = 0.f;
                    for (int pi = 0; pi < BCHUNK / AGAVE_PAGE; ++pi) {
                        const long vp = page_of[pi];
                        if (vp < 0) continue;
                        const T* vblk = v_pages + ((size_t)vp * nkv + kvh) * vd * AGAVE_PAGE;
                        const T* vr = vblk + (size_t)d * AGAVE_PAGE;
                        for (int r = 0; r < AGAVE_PAGE; ++r) {
                            const float w = sc[pi * AGAVE_PAGE + r];
                            if (w != 0.f) sum = fmaf(w, ld(A.packed ? vblk + v_operand_at(d, r) : vr + r), sum);   // rows out of range hold w == 0
                        }
                    }
                    acc[a] = acc[a] * alpha + sum;
                }
            }
            __syncthreads();     // sc[] and page_of[] are rewritten by the next pass
        }
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    T* out = (T*)A.out;
    const T* gate = (const T*)A.gate;
#pragma unroll
    for (int a = 0; a < BACC; ++a) {
        const int d = tid + a * 256;
        if (d < vd) {
            float y = acc[a] * inv;
            if (gate) y *= 1.0f / (1.0f + expf(-ld(gate + (size_t)t * A.ldg + (size_t)h * vd + d)));
            st(out + (size_t)t * A.ldo + (size_t)h * vd + d, y);
        }
    }
}

static int check_biased(const BiasedArgs& A, int N) {
    AGAVE_CHECK(N >= 0 && A.nh > 0 && A.nkv > 0 && A.hd > 0 && A.vd > 0, "attn_biased: bad sizes N=%d nh=%d nkv=%d hd=%d vd=%d", N,
                A.nh, A.nkv, A.hd, A.vd);
    AGAVE_CHECK(A.nh % A.nkv == 0, "attn_biased: %d query heads are not a multiple of %d kv heads", A.nh, A.nkv);
    AGAVE_CHECK(A.hd <= 1024 && A.vd <= 256 * BACC, "attn_biased: head sizes %d / %d exceed 1024", A.hd, A.vd);
    AGAVE_CHECK(A.ldq >= (long)A.nh * A.hd && A.ldo >= (long)A.nh * A.vd && (!A.gate || A.ldg >= (long)A.nh * A.vd),
                "attn_biased: a row stride is too small");
    AGAVE_CHECK(A.window >= 0 && A.keep_first >= 0 && A.head >= 0, "attn_biased: negative window, kept positions or kept pages");
    AGAVE_CHECK(A.chunk >= 0 && A.softcap >= 0.f && (A.chunk == 0 || A.keep_first == 0), "attn_biased: a negative chunk or cap, or chunks with kept first positions");
    AGAVE_CHECK(A.keep_first <= A.head * AGAVE_PAGE, "attn_biased: %d kept positions do not fit %d kept pages", A.keep_first, A.head);
    AGAVE_CHECK(A.bias_mode >= 0 && A.bias_mode <= 2 && (A.bias_mode == 0 || A.bias) && (A.bias_mode != 2 || A.bias_len > 0),
                "attn_biased: bias mode %d without its numbers", A.bias_mode);
    AGAVE_CHECK(A.q && A.out && A.k_pages && A.v_pages && A.table && A.base && A.tok_seq && A.tok_pos && A.width > 0 && A.n_pages > 0,
                "attn_biased: null buffer or empty table");
    AGAVE_CHECK((long)N * A.nh < 2147483647L, "attn_biased: too many (token, head) pairs");
    return 0;
}

extern "C" int agave_attn_biased_plain(int dtype, const void* q, long ldq, void* out, long ldo, const void* gate, long ldg,
                                       const void* k_pages, const void* v_pages, const int* table, int width,
                                       const int* base, int head, int n_pages, const int* tok_seq, const int* tok_pos, int N,
                                       int nh, int nkv, int hd, int vd, float scale, int window, int keep_first,
                                       int bias_mode, const float* bias, int bias_len, const float* sink, int packed,
                                       int chunk, float softcap, hipStream_t stream) {
    BiasedArgs A{q, ldq, out, ldo, gate, ldg, k_pages, v_pages, table, width, base, head, n_pages, tok_seq, tok_pos,
                 nh, nkv, hd, vd, scale, window, keep_first, bias_mode, bias, bias_len, sink, packed, chunk, softcap};
    AGAVE_CHECK(!packed || dtype == AGAVE_BF16, "attn_biased: pages in operand order hold bfloat16");
    if (check_biased(A, N)) return -1;
    if (N == 0) return 0;
    if (dtype == AGAVE_F32)
        attn_biased_plain_kernel<float><<<N * nh, 256, 0, stream>>>(A);
    else if (dtype == AGAVE_BF16)
        attn_biased_plain_kernel<bf16><<<N * nh, 256, 0, stream>>>(A);
    else
        AGAVE_CHECK(false, "attn_biased: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("attn_biased_plain");
    return 0;
}

// ------------------------------------------------------------------ matrix-core kernel (bfloat16)
// A wave owns NC blocks of 16 "columns": in a step of many rows, 16 NC query rows of one head; in a step of
// one row a sequence, the row's query heads of one key head (the heads of a group read the same keys).  Per
// page of 64 keys it computes the transposed scores S^T = K Q^T (keys x columns) with
// v_mfma_f32_16x16x32_bf16, so that a lane holds scores of one column a block only: the column's running
// maximum, sum and rescaling factor are the lane's own (and its three partners' in the other lane
// groups), and the probabilities go from the score registers straight into the B operand of
// O^T += V^T P^T.  A key or value operand that was loaded serves all NC column blocks.
// Which key a row of a score tile stands for is the kernel's choice; row i of key block kb is key
//   key_of(kb, i) = 32 (kb / 2) + 8 (i / 4) + 4 (kb % 2) + i % 4
// of the page, so that a lane group's scores of two neighbouring key blocks are eight neighbouring keys, the
// eight that a lane's B operand of one step of O^T += V^T P^T holds, and the matching A operand is 16 bytes
// of a value column's row in the transposed page:
//   S^T tile of key block kb: lane l holds keys 32 (kb / 2) + 8 (l / 16) + 4 (kb % 2) + e, e = 0..3, of column l % 16
//   O^T block nb:             lane l holds value columns 16 nb + 4 (l / 16) + e of column l % 16
// Many rows: a workgroup is four waves with 16 NC rows each, all pages each.  One row: the workgroup's
// waves (four or eight) share the pages of one (row, key head) and wave 0 merges their partial results
// through LDS.  KS = ceil(hd / 32) steps along the head, VB = blocks of 16 value columns (sizes are
// padded with zeros in registers, never in memory).
struct MfmaMode {
    int one_row;                 // 1: a step of one row a sequence
    const int* cu;               // [sequences + 1] first row of every sequence (many rows)
    int table_in_lds;            // the bias table's row of this head is copied to LDS (many rows)
    int splits;                  // one row: this many workgroups share a row's pages and leave partial results
    float* parts;                // [rows][heads][splits][2 + vd]: reference, sum, unnormalised row (splits > 1)
    int q_off;                   // floats of LDS in front of the place for Q (the longest heads keep Q there)
};

typedef __attribute__((address_space(3))) u32x4_t lds_u32x4;

// (Heads of more than 256 key or value elements hold most of a wave's registers in Q and O^T: their workgroups have
// four waves, one a SIMD, and a wave may use the whole register file.)
template <int KS, int VB, int NC, bool LDSP>
__global__ __launch_bounds__((KS > 8 || VB > 16) ? 256 : 512) void attn_biased_mfma_kernel(BiasedArgs A, MfmaMode M) {
    extern __shared__ float lds_generic[];
    // (every LDS access goes through a pointer that says so: no pointer may end up chosen between the two memories)
    typedef __attribute__((address_space(3))) float lds_float;
    lds_float* lds = (lds_float*)lds_generic;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int nh = A.nh, nkv = A.nkv, hd = A.hd, vd = A.vd;
    const int per = nh / nkv;
    constexpr int WROWS = 16 * NC;                  // rows a wave in a step of many rows

    // my columns (one a block): row, position, whether it exists; the head is the same for all in a step of many rows
    int row[NC], pos[NC], head, b;
    bool valid[NC];
    int pmin, pmax;                                 // the wave's range of positions (the same in every lane)
    int wg_first = 0, wg_last = 0;                  // the workgroup's (many rows)
    bool wave_on = true;
    const int splits = M.one_row ? M.splits : 1, sp = M.one_row ? (int)(blockIdx.x % splits) : 0;
    if (M.one_row) {
        row[0] = blockIdx.x / splits;
        b = A.tok_seq[row[0]];
        const int hg = blockIdx.z * 16 + c;
        valid[0] = hg < per;
        head = blockIdx.y * per + (valid[0] ? hg : 0);
        pos[0] = A.tok_pos[row[0]];
        pmin = pmax = pos[0];
#pragma unroll
        for (int cb = 1; cb < NC; ++cb) {           // (one block of columns in this mode)
            row[cb] = row[0];
            pos[cb] = pos[0];
            valid[cb] = false;
        }
    } else {
        b = blockIdx.y;
        const int r0 = M.cu[b] + blockIdx.x * 4 * WROWS, r1 = M.cu[b + 1];
        if (r0 >= r1) return;                                   // (the whole workgroup: a shorter sequence of the batch)
        head = blockIdx.z;
        if (M.table_in_lds) {                                   // (before any wave leaves: all of them meet at the barrier)
            const float* src = A.bias + (size_t)head * A.bias_len;
            for (int i = threadIdx.x; i < A.bias_len; i += blockDim.x) lds[i] = src[i] * 1.4426950408889634f;
            __syncthreads();
        }
        const int wr0 = r0 + w * WROWS;
        wave_on = wr0 < r1;
        if (!LDSP && !wave_on) return;                          // this wave has no rows (with pages through LDS it still carries them)
#pragma unroll
        for (int cb = 0; cb < NC; ++cb) {
            row[cb] = wr0 + 16 * cb + c;
            valid[cb] = row[cb] < r1;
            if (!valid[cb]) row[cb] = r1 - 1;
            pos[cb] = A.tok_pos[row[cb]];
        }
        pmin = A.tok_pos[wave_on ? wr0 : r1 - 1];
        pmax = A.tok_pos[min(wr0 + WROWS, r1) - 1];
        wg_first = A.tok_pos[r0];
        wg_last = A.tok_pos[min(r0 + 4 * WROWS, r1) - 1];
    }
    const int kvh = head / per;
    const int ksl = (hd + 31) / 32;                 // steps along the head that the pages hold
    const int W = A.window, keep = A.keep_first, C = A.chunk;
    int lo = W > 0 ? max(0, pmin - W + 1) : 0;
    if (C > 0) lo = max(lo, (pmin / C) * C);           // (the earliest chunk start among the wave's rows)
    int cstart[NC];                                     // first position of each column's chunk
#pragma unroll
    for (int cb = 0; cb < NC; ++cb) cstart[cb] = C > 0 ? (pos[cb] / C) * C : 0;
    const int cstart_max = C > 0 ? (pmax / C) * C : 0;
    const float cap2 = A.softcap * 1.4426950408889634f, scale_cap = A.softcap > 0.f ? A.scale / A.softcap : 0.f;
    const int first_win = lo / AGAVE_PAGE;
    const int n_kept = min(first_win, (keep + AGAVE_PAGE - 1) / AGAVE_PAGE);
    const int n_pg = n_kept + pmax / AGAVE_PAGE - first_win + 1;
    const int pbase = A.base[b];

    const float LOG2E = 1.4426950408889634f;
    const float* bias_row = nullptr;           // table of my head
    const float scale2 = A.scale * LOG2E;
    const float slope2 = A.bias_mode == 1 ? A.bias[head] * LOG2E : 0.f;
    if (A.bias_mode == 2) bias_row = A.bias + (size_t)head * A.bias_len;

    // Q as the B operand: lane holds Q[column c][32 ks + 8 g .. + 8]
    // The longest heads (more than 12 steps) keep Q in LDS instead, in the same order, and read an operand when it is
    // multiplied: with O^T of 512 value columns in registers there is no room for both.  A wave reads what it wrote
    // itself (in a step of one row all waves hold the same Q and write the same place).
    constexpr bool QL = KS > 12;
    static_assert(!QL || NC == 1, "Q in LDS is for one block of columns a wave");
    lds_u32x4* qs = (lds_u32x4*)(lds + M.q_off) + (M.one_row ? 0 : (size_t)w * KS * 64);
    frag16 qf[NC][QL ? 1 : KS];
#pragma unroll
    for (int cb = 0; cb < NC; ++cb) {
        const bf16* qrow = (const bf16*)A.q + (size_t)row[cb] * A.ldq + (size_t)head * hd;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            // (every load is written without a condition, from an address inside the row, and emptied afterwards
            // where it lies past the head's end: a load under a per-lane condition is waited for on the spot)
            const int k0 = 32 * ks + 8 * g;
            const uint4 got = *reinterpret_cast<const uint4*>(qrow + (k0 < hd ? k0 : 0));
            frag16 f;
            f.u = (valid[cb] && k0 < hd) ? got : make_uint4(0, 0, 0, 0);
            if constexpr (QL) qs[ks * 64 + lane] = f.r;
            else qf[cb][ks] = f;
        }
    }

    f32x4_t o[NC][VB];
    float m[NC], l[NC];
#pragma unroll
    for (int cb = 0; cb < NC; ++cb) {
#pragma unroll
        for (int nb = 0; nb < VB; ++nb) o[cb][nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        m[cb] = -INFINITY;
        l[cb] = 0.f;
        if (A.sink && (!M.one_row || (w == 0 && sp == 0))) {
            m[cb] = A.sink[head] * LOG2E;
            l[cb] = g == 0 ? 1.f : 0.f;         // the lane groups' sums are added up at the end
        }
    }

    const int stride = M.one_row ? nw * splits : 1;
    auto page_of = [&](int idx) -> long {
        if (idx >= n_pg) return -1;
        const int pi = idx < n_kept ? idx : first_win + idx - n_kept;
        const int col = page_col(pi, pbase, A.head);
        const long pg = (col >= 0 && col < A.width) ? A.table[(size_t)b * A.width + col] : -1;
        return pg < A.n_pages ? pg : -1;
    };
    // One page: kt and vt hold its key and value operands, 64 lanes x 16 bytes each (tile (kb, ks) of the keys at
    // kb ksl + ks, tile (nb, h) of the values at 2 nb + h), in memory or in LDS.
    auto page = [&](int pi, auto kt, auto vt) {
        // What the page needs from memory is asked for before any of it is used (a wave's loads come back in the
        // order they left): the bias where it is read from memory, the value operands where the registers allow, then
        // the keys.
        constexpr bool V_AHEAD = VB <= 8 && NC == 1;
        float bv[NC][4][4];
        if (A.bias_mode == 2 && !M.table_in_lds) {
#pragma unroll
            for (int cb = 0; cb < NC; ++cb)
#pragma unroll
                for (int kb = 0; kb < 4; ++kb)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int dist = pos[cb] - (pi * AGAVE_PAGE + 32 * (kb >> 1) + 8 * g + 4 * (kb & 1) + e);
                        bv[cb][kb][e] = bias_row[dist < 0 ? 0 : (dist < A.bias_len ? dist : A.bias_len - 1)] * LOG2E;
                    }
        }
        frag16 va[V_AHEAD ? VB : 1][2];
        if (V_AHEAD) {
#pragma unroll
            for (int nb = 0; nb < VB; ++nb) {
                // (a block past the value size reads the first block again and is not used)
#pragma unroll
                for (int h2 = 0; h2 < 2; ++h2) va[V_AHEAD ? nb : 0][h2].r = vt[((16 * nb < vd ? nb : 0) * 2 + h2) * 64 + lane];
            }
        }
        // scores of the page's four key blocks
        f32x4_t s[NC][4];
        if constexpr (KS > 9 && !QL) {
            // A long head: the page's 4 KS key operands in chunks of four, a chunk asked for while the one before it is
            // multiplied (two sets of registers that take turns).  The compiler is told not to move anything across
            // a chunk's border: left alone it asks for everything at once and runs out of registers, and a loop that
            // waits for every chunk before it asks for the next is a chain of round trips to memory.
            constexpr int C = 4, NCH = (4 * KS + C - 1) / C;
            frag16 kbuf[2][C];
#pragma unroll
            for (int cb = 0; cb < NC; ++cb)
#pragma unroll
                for (int kb = 0; kb < 4; ++kb) s[cb][kb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ch = -1; ch < NCH; ++ch) {
                if (ch + 1 < NCH) {
#pragma unroll
                    for (int i = 0; i < C; ++i) {
                        const int e = (ch + 1) * C + i;
                        if (e < 4 * KS) {
                            const int kb = e / KS, ks = e % KS;
                            const u32x4_t got = kt[(kb * ksl + (ks < ksl ? ks : 0)) * 64 + lane];
                            kbuf[(ch + 1) & 1][i].r = ks < ksl ? got : u32x4_t{0u, 0u, 0u, 0u};
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if (ch >= 0) {
#pragma unroll
                    for (int i = 0; i < C; ++i) {
                        const int e = ch * C + i;
                        if (e < 4 * KS) {
                            const int kb = e / KS, ks = e % KS;
#pragma unroll
                            for (int cb = 0; cb < NC; ++cb) {
                                s[cb][kb] = mfma_16x16x32(kbuf[ch & 1][i], qf[cb][ks], s[cb][kb]);
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        } else {
#pragma unroll
            for (int kb = 0; kb < 4; ++kb) {
                // (a whole operand in one load of a kilobyte; steps past the head's end read step 0 again and are
                // emptied.  The longest heads, which have no registers left for a second set of operands, take their
                // steps in three batches that wait for each other.)
                constexpr int KCH = QL ? 6 : KS;
#pragma unroll
                for (int cb = 0; cb < NC; ++cb) s[cb][kb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int k0 = 0; k0 < KS; k0 += KCH) {
                    frag16 kf[KCH];
#pragma unroll
                    for (int kk = 0; kk < KCH; ++kk) {
                        const int ks = k0 + kk;
                        const u32x4_t got = kt[(kb * ksl + (ks < ksl ? ks : 0)) * 64 + lane];
                        kf[kk].r = ks < ksl ? got : u32x4_t{0u, 0u, 0u, 0u};
                    }
#pragma unroll
                    for (int cb = 0; cb < NC; ++cb) {
#pragma unroll
                        for (int kk = 0; kk < KCH; ++kk)
                            if (k0 + kk < KS) {
                                frag16 qv;
                                if constexpr (QL) qv.r = qs[(k0 + kk) * 64 + lane];
                                else qv = qf[cb][QL ? 0 : k0 + kk];
                                s[cb][kb] = mfma_16x16x32(kf[kk], qv, s[cb][kb]);
                            }
                    }
                    if constexpr (QL) __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        // Scale, bias, mask and softmax, a column block at a time, in the base-2 domain (scale, slopes, table and
        // sinks carry the factor log2(e), so an exponential is one instruction).  A page that every row of the wave
        // sees whole (below the diagonal, inside the window or among the kept positions) needs no mask: most pages
        // of a long sequence are such, and the mask is most of the arithmetic of a score.
        frag16 pf[NC][2];
        float alpha[NC];
        const int j_last = pi * AGAVE_PAGE + AGAVE_PAGE - 1;
        const bool whole = j_last <= pmin && (W == 0 || pmax - pi * AGAVE_PAGE < W || j_last < keep) &&
                           (C == 0 || pi * AGAVE_PAGE >= cstart_max);
        auto scores = [&](auto whole_tag, auto table_tag) {
            constexpr bool WHOLE = decltype(whole_tag)::value != 0, TABLE = decltype(table_tag)::value != 0;
#pragma unroll
            for (int cb = 0; cb < NC; ++cb) {
                float tile_max = -INFINITY;
                const int d0 = pos[cb] - pi * AGAVE_PAGE - 8 * g;           // distance to the lane group's first key
                const float t0 = -slope2 * (float)d0;
#pragma unroll
                for (int kb = 0; kb < 4; ++kb) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int off = 32 * (kb >> 1) + 4 * (kb & 1) + e;  // (a constant once the loops are unrolled)
                        const int dist = d0 - off;
                        float v;
                        if (cap2 > 0.f) {
                            // cap tanh(x / cap) with tanh(z) = 1 - 2 / (e^(2z) + 1), which is right at both ends
                            const float e2 = __builtin_amdgcn_exp2f(s[cb][kb][e] * scale_cap * 2.8853900817779268f);
                            v = fmaf(cap2, 1.0f - 2.0f * __builtin_amdgcn_rcpf(e2 + 1.0f), fmaf(slope2, (float)off, t0));
                        } else {
                            v = fmaf(s[cb][kb][e], scale2, fmaf(slope2, (float)off, t0));
                        }
                        bool see = true;
                        if (!WHOLE) see = valid[cb] && dist >= 0 && (W == 0 || dist < W || pos[cb] - dist < keep) &&
                                          pos[cb] - dist >= cstart[cb];
                        if (TABLE) {
                            int at = dist < A.bias_len ? dist : A.bias_len - 1;
                            if (!WHOLE) at = see ? at : 0;
                            v += M.table_in_lds ? lds[at] : bv[cb][kb][e];
                        }
                        if (!WHOLE) v = see ? v : -INFINITY;
                        s[cb][kb][e] = v;
                        tile_max = fmaxf(tile_max, v);
                    }
                }
                tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16));
                tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32));
                const float m_new = fmaxf(m[cb], tile_max);
                // (a column that sees nothing of this page and has seen nothing before keeps m = -inf; its p are 0)
                const float ref = m_new == -INFINITY ? 0.f : m_new;
                alpha[cb] = m[cb] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[cb] - ref);
                float sum = 0.f;
#pragma unroll
                for (int kb = 0; kb < 4; ++kb) {
                    float p[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        p[e] = __builtin_amdgcn_exp2f(s[cb][kb][e] - ref);      // 2^(-inf) = 0 for what is not seen
                        sum += p[e];
                    }
                    const uint32_t lo2 = f32x2_to_bf16x2(p[0], p[1]), hi2 = f32x2_to_bf16x2(p[2], p[3]);
                    if (kb & 1) {
                        pf[cb][kb >> 1].r[2] = lo2;
                        pf[cb][kb >> 1].r[3] = hi2;
                    } else {
                        pf[cb][kb >> 1].r[0] = lo2;
                        pf[cb][kb >> 1].r[1] = hi2;
                    }
                }
                l[cb] = l[cb] * alpha[cb] + sum;
                m[cb] = m_new;
            }
        };
        if (A.bias_mode == 2) {
            if (whole) scores(IntC<1>{}, IntC<1>{}); else scores(IntC<0>{}, IntC<1>{});
        } else {
            if (whole) scores(IntC<1>{}, IntC<0>{}); else scores(IntC<0>{}, IntC<0>{});
        }
        // O^T = O^T alpha + V^T P^T
        if constexpr (VB > 16 && !QL) {
            // (wide values: two blocks' operands at a time, the next two asked for while these are multiplied)
            constexpr int VG = 2, NVG = VB / VG;
            frag16 vbuf[2][VG][2];
#pragma unroll
            for (int gi = -1; gi < NVG; ++gi) {
                if (gi + 1 < NVG) {
#pragma unroll
                    for (int j = 0; j < VG; ++j) {
                        const int nb = (gi + 1) * VG + j, nbl = 16 * nb < vd ? nb : 0;     // (a block past the value size reads the first again)
#pragma unroll
                        for (int h2 = 0; h2 < 2; ++h2) vbuf[(gi + 1) & 1][j][h2].r = vt[(nbl * 2 + h2) * 64 + lane];
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if (gi >= 0) {
#pragma unroll
                    for (int j = 0; j < VG; ++j) {
                        const int nb = gi * VG + j;
                        if (16 * nb < vd) {
#pragma unroll
                            for (int cb = 0; cb < NC; ++cb) {
                                o[cb][nb] *= alpha[cb];
                                o[cb][nb] = mfma_16x16x32(vbuf[gi & 1][j][0], pf[cb][0], o[cb][nb]);
                                o[cb][nb] = mfma_16x16x32(vbuf[gi & 1][j][1], pf[cb][1], o[cb][nb]);
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        } else {
#pragma unroll
        for (int nb = 0; nb < VB; ++nb) {
            if (16 * nb < vd) {
                frag16 vf[2];
                if (V_AHEAD) {
                    vf[0] = va[V_AHEAD ? nb : 0][0];
                    vf[1] = va[V_AHEAD ? nb : 0][1];
                } else {
#pragma unroll
                    for (int h2 = 0; h2 < 2; ++h2) vf[h2].r = vt[(nb * 2 + h2) * 64 + lane];
                }
#pragma unroll
                for (int cb = 0; cb < NC; ++cb) {
                    o[cb][nb] *= alpha[cb];
                    o[cb][nb] = mfma_16x16x32(vf[0], pf[cb][0], o[cb][nb]);
                    o[cb][nb] = mfma_16x16x32(vf[1], pf[cb][1], o[cb][nb]);
                }
            }
            if constexpr (QL) {                         // (four blocks' value operands at a time, see the keys)
                if ((nb & 3) == 3) __builtin_amdgcn_sched_barrier(0);
            }
        }
        }
    };

    if constexpr (LDSP) {
        // Many rows, pages through LDS: the workgroup's four waves (one head, 64 NC rows) bring every page they need
        // between them into LDS once, straight from memory and a page ahead of the one being multiplied, in two
        // buffers that take turns; a wave multiplies the pages its own rows see.
        const int tbl = M.table_in_lds ? (A.bias_len + 3) / 4 * 4 : 0;         // floats in front of the pages
        lds_u32x4* pages = (lds_u32x4*)(lds + tbl);
        const int n_k = 4 * ksl, n_v = (vd / 16) * 2, buf_tiles = n_k + n_v;
        int g_lo = W > 0 ? max(0, wg_first - W + 1) : 0;
        if (C > 0) g_lo = max(g_lo, (wg_first / C) * C);
        const int g_first = g_lo / AGAVE_PAGE;
        const int g_kept = min(g_first, (keep + AGAVE_PAGE - 1) / AGAVE_PAGE);
        const int g_n = g_kept + wg_last / AGAVE_PAGE - g_first + 1;
        auto page_at = [&](int gi, int& pi) -> long {
            pi = gi < g_kept ? gi : g_first + gi - g_kept;
            const int col = page_col(pi, pbase, A.head);
            const long pg = (col >= 0 && col < A.width) ? A.table[(size_t)b * A.width + col] : -1;
            return pg < A.n_pages ? pg : -1;
        };
        auto fetch = [&](int gi, int buf) {
            int pi;
            const long pg = page_at(gi, pi);
            if (pg < 0) return;
            const uint4* ksrc = (const uint4*)A.k_pages + ((size_t)pg * nkv + kvh) * (size_t)n_k * 64;
            const uint4* vsrc = (const uint4*)A.v_pages + ((size_t)pg * nkv + kvh) * (size_t)n_v * 64;
            for (int ti = w; ti < buf_tiles; ti += 4) {
                const uint4* src = ti < n_k ? ksrc + (size_t)ti * 64 : vsrc + (size_t)(ti - n_k) * 64;
                lds_u32x4* dst = pages + ((size_t)buf * buf_tiles + ti) * 64;
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + lane),
                                                 (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
            }
        };
        fetch(0, 0);
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        for (int gi = 0; gi < g_n; ++gi) {
            const int buf = gi & 1;
            if (gi + 1 < g_n) fetch(gi + 1, buf ^ 1);
            int pi;
            const long pg = page_at(gi, pi);
            const bool mine = wave_on && pg >= 0 && pi <= pmax / AGAVE_PAGE && (pi >= first_win || pi * AGAVE_PAGE < keep);
            if (mine) {
                const lds_u32x4* kl = pages + (size_t)buf * buf_tiles * 64;
                page(pi, kl, kl + (size_t)n_k * 64);
            }
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
        }
        if (!wave_on) return;
    } else {
        int idx = M.one_row ? sp * nw + w : 0;
        long pg = page_of(idx);
        for (; idx < n_pg; idx += stride) {
            const long pg_next = page_of(idx + stride);         // asked for now, used in the next turn
            const long pg_now = pg;
            pg = pg_next;
            if (pg_now < 0) continue;
            const int pi = idx < n_kept ? idx : first_win + idx - n_kept;
            const u32x4_t* kt = (const u32x4_t*)A.k_pages + ((size_t)pg_now * nkv + kvh) * (size_t)ksl * 4 * 64;
            const u32x4_t* vt = (const u32x4_t*)A.v_pages + ((size_t)pg_now * nkv + kvh) * (size_t)(vd / 16) * 2 * 64;
            page(pi, kt, vt);
        }
    }
    // the columns' sums over the four lane groups
#pragma unroll
    for (int cb = 0; cb < NC; ++cb) {
        l[cb] += __shfl_xor(l[cb], 16);
        l[cb] += __shfl_xor(l[cb], 32);
    }

    if (M.one_row) {
        // the other waves leave (m, l, O^T) in LDS; wave 0 merges
        const int per_wave = VB * 16 * 16 + 32;
        if (w > 0) {
            lds_float* mine = lds + (size_t)(w - 1) * per_wave;
            if (g == 0) {
                mine[c] = m[0];
                mine[16 + c] = l[0];
            }
#pragma unroll
            for (int nb = 0; nb < VB; ++nb)
#pragma unroll
                for (int e = 0; e < 4; ++e) mine[32 + (16 * nb + 4 * g + (e ^ (g & 1))) * 16 + c] = o[0][nb][e];     // (odd lane groups swap neighbours: no two lanes of a half wave share a bank)
        }
        __syncthreads();
        if (w > 0) return;
        for (int ow = 0; ow < nw - 1; ++ow) {
            const lds_float* other = lds + (size_t)ow * per_wave;
            const float m2 = other[c], l2 = other[16 + c];
            if (m2 == -INFINITY) continue;                      // (per lane: that wave saw nothing for my column)
            const float m_new = fmaxf(m[0], m2);
            const float a1 = m[0] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[0] - m_new), a2 = __builtin_amdgcn_exp2f(m2 - m_new);
            l[0] = l[0] * a1 + l2 * a2;
            m[0] = m_new;
#pragma unroll
            for (int nb = 0; nb < VB; ++nb) {
#pragma unroll
                for (int e = 0; e < 4; ++e) o[0][nb][e] = o[0][nb][e] * a1 + other[32 + (16 * nb + 4 * g + (e ^ (g & 1))) * 16 + c] * a2;
                if constexpr (VB > 16) {                // (or all of the other wave's row is read before any of it is used)
                    if ((nb & 3) == 3) __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        if (splits > 1) {
            // this workgroup's share of the row: reference, sum and the unnormalised sums over the values
            if (!valid[0]) return;
            float* mine = M.parts + (((size_t)row[0] * nh + head) * splits + sp) * (size_t)(vd + 2);
            if (g == 0) {
                mine[0] = m[0];
                mine[1] = l[0];
            }
#pragma unroll
            for (int nb = 0; nb < VB; ++nb) {
                const int d0 = 16 * nb + 4 * g;
                if (d0 < vd) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) mine[2 + d0 + e] = o[0][nb][e];
                }
            }
            return;
        }
    }
#pragma unroll
    for (int cb = 0; cb < NC; ++cb) {
        if (!valid[cb]) continue;
        const float inv = l[cb] > 0.f ? 1.0f / l[cb] : 0.f;
        bf16* orow = (bf16*)A.out + (size_t)row[cb] * A.ldo + (size_t)head * vd;
        const bf16* grow = A.gate ? (const bf16*)A.gate + (size_t)row[cb] * A.ldg + (size_t)head * vd : nullptr;
#pragma unroll
        for (int nb = 0; nb < VB; ++nb) {
            const int d0 = 16 * nb + 4 * g;
            if (d0 < vd) {
                float y[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    y[e] = o[cb][nb][e] * inv;
                    if (grow) y[e] *= 1.0f / (1.0f + __expf(-bf16_to_f32(grow[d0 + e])));
                }
                uint2 packed;
                packed.x = f32x2_to_bf16x2(y[0], y[1]);
                packed.y = f32x2_to_bf16x2(y[2], y[3]);
                *reinterpret_cast<uint2*>(orow + d0) = packed;
            }
        }
    }
}

// The shares of a row that several workgroups left: a workgroup per (row, head), a thread per value column.
__global__ __launch_bounds__(256) void attn_biased_merge_kernel(const float* __restrict__ parts, int splits, int nh, int vd,
                                                                bf16* __restrict__ out, long ldo, const bf16* __restrict__ gate,
                                                                long ldg) {
    const int t = blockIdx.x / nh, h = blockIdx.x % nh;
    const float* mine = parts + (size_t)blockIdx.x * splits * (vd + 2);
    float mx = -INFINITY;
    for (int s = 0; s < splits; ++s) mx = fmaxf(mx, mine[(size_t)s * (vd + 2)]);
    float total = 0.f;
    for (int s = 0; s < splits; ++s) {
        const float ms = mine[(size_t)s * (vd + 2)];
        if (ms != -INFINITY) total += mine[(size_t)s * (vd + 2) + 1] * __builtin_amdgcn_exp2f(ms - mx);
    }
    const float inv = total > 0.f ? 1.0f / total : 0.f;
    for (int d = threadIdx.x; d < vd; d += blockDim.x) {
        float acc = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float ms = mine[(size_t)s * (vd + 2)];
            if (ms != -INFINITY) acc = fmaf(mine[(size_t)s * (vd + 2) + 2 + d], __builtin_amdgcn_exp2f(ms - mx), acc);
        }
        float y = acc * inv;
        if (gate) y *= 1.0f / (1.0f + __expf(-bf16_to_f32(gate[(size_t)t * ldg + (size_t)h * vd + d])));
        out[(size_t)t * ldo + (size_t)h * vd + d] = f32_to_bf16(y);
    }
}

template <int KS, int VB>
static int launch_biased_mfma(const BiasedArgs& A, const MfmaMode& M, dim3 grid, int threads, int nc, size_t lds_bytes,
                              hipStream_t stream) {
    if (nc == 2) {
        if constexpr (VB <= 8) {
            static bool raised = false;             // (the two page buffers and the table may need more LDS than a kernel gets unasked)
            if (!raised) {
                AGAVE_CHECK(hipFuncSetAttribute((const void*)attn_biased_mfma_kernel<KS, VB, 2, true>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024) == hipSuccess,
                            "attn_biased_mfma: cannot raise the LDS allowance");
                raised = true;
            }
            attn_biased_mfma_kernel<KS, VB, 2, true><<<grid, threads, lds_bytes, stream>>>(A, M);
        }
    } else {
        if (lds_bytes > 64 * 1024) {
            static bool raised1 = false;            // (the waves' partial results of a wide value head)
            if (!raised1) {
                AGAVE_CHECK(hipFuncSetAttribute((const void*)attn_biased_mfma_kernel<KS, VB, 1, false>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024) == hipSuccess,
                            "attn_biased_mfma: cannot raise the LDS allowance");
                raised1 = true;
            }
        }
        attn_biased_mfma_kernel<KS, VB, 1, false><<<grid, threads, lds_bytes, stream>>>(A, M);
    }
    return 0;
}

#define BIASED_VB(KS_)                                                                                   \
    switch (vb) {                                                                                        \
        case 2: rc = launch_biased_mfma<KS_, 2>(A, M, grid, threads, nc, lds_bytes, stream); break;      \
        case 4: rc = launch_biased_mfma<KS_, 4>(A, M, grid, threads, nc, lds_bytes, stream); break;      \
        case 8: rc = launch_biased_mfma<KS_, 8>(A, M, grid, threads, nc, lds_bytes, stream); break;      \
        default: rc = launch_biased_mfma<KS_, 16>(A, M, grid, threads, nc, lds_bytes, stream); break;    \
    }

// 1 if the matrix-core kernel takes these sizes (the caller then may call it), else 0
extern "C" int agave_attn_biased_mfma_ok(int hd, int vd, int ldq, int ldo, int ldg) {
    return (hd % 8 == 0 && hd <= 576 && vd % 16 == 0 && vd <= 512 && ldq % 8 == 0 && ldo % 4 == 0 && ldg % 4 == 0) ? 1 : 0;
}

// `cu`: first row of every sequence (device, sequences + 1 entries), used by steps of many rows;
// `max_rows`: the most rows a sequence brings; `one_row`: every sequence brings one row.
extern "C" int agave_attn_biased_mfma(const void* q, long ldq, void* out, long ldo, const void* gate, long ldg,
                                      const void* k_pages, const void* v_pages, const int* table, int width, const int* base,
                                      int head, int n_pages, const int* tok_seq, const int* tok_pos, const int* cu, int N,
                                      int n_seqs, int max_rows, int one_row, int nh, int nkv, int hd, int vd, float scale,
                                      int window, int keep_first, int bias_mode, const float* bias, int bias_len,
                                      const float* sink, int splits, float* parts, int chunk, float softcap,
                                      hipStream_t stream) {
    BiasedArgs A{q, ldq, out, ldo, gate, ldg, k_pages, v_pages, table, width, base, head, n_pages, tok_seq, tok_pos,
                 nh, nkv, hd, vd, scale, window, keep_first, bias_mode, bias, bias_len, sink, 1, chunk, softcap};
    if (check_biased(A, N)) return -1;
    AGAVE_CHECK(splits >= 1 && splits <= 64 && (splits == 1 || (one_row && parts)),
                "attn_biased_mfma: %d shares of a row (1 to 64, in steps of one row a sequence, with memory for them)", splits);
    AGAVE_CHECK(agave_attn_biased_mfma_ok(hd, vd, (int)(ldq % 8), (int)(ldo % 4), (int)(ldg % 4)),
                "attn_biased_mfma: head sizes %d / %d or row strides that the matrix-core kernel does not take", hd, vd);
    AGAVE_CHECK(((uintptr_t)q % 16) == 0 && ((uintptr_t)out % 8) == 0 && ((uintptr_t)gate % 8) == 0 && (nh * (long)hd) % 8 == 0,
                "attn_biased_mfma: rows must be aligned to 16 bytes");
    AGAVE_CHECK(cu && n_seqs > 0 && max_rows > 0 && (!one_row || N == n_seqs), "attn_biased_mfma: bad step");
    if (N == 0) return 0;
    // (heads beyond 256 come in two sizes of both at once: up to 384 / 384 and up to 576 / 512)
    const bool wide = hd > 256 || vd > 256, widest = hd > 384 || vd > 384;
    const int ks = wide ? (widest ? 18 : 12) : hd <= 32 ? 1 : hd <= 64 ? 2 : hd <= 128 ? 4 : 8;
    const int vb = wide ? (widest ? 32 : 24) : vd <= 32 ? 2 : vd <= 64 ? 4 : vd <= 128 ? 8 : 16;
    MfmaMode M{one_row, cu, 0, splits, parts, 0};
    dim3 grid;
    size_t lds_bytes = 0;
    int threads = 256, nc = 1;
    if (one_row) {
        // eight waves share a row's pages where their partial results fit the LDS, else four
        const int per = nh / nkv;
        const int nw = vb <= 8 ? 8 : 4;
        threads = 64 * nw;
        grid = dim3(N * splits, nkv, (per + 15) / 16);
        lds_bytes = (size_t)(nw - 1) * (vb * 16 * 16 + 32) * sizeof(float);
    } else {
        // 32 rows a wave where the step is long enough to fill the chip that way and the registers allow
        // (then the workgroup's waves share a head's pages through LDS)
        nc = (vb <= 8 && (long)((max_rows + 127) / 128) * n_seqs * nh >= 256) ? 2 : 1;
        if (bias_mode == 2 && bias_len <= 8192) {
            M.table_in_lds = 1;
            lds_bytes = (size_t)((bias_len + 3) / 4 * 4) * sizeof(float);
        }
        if (nc == 2) {
            const size_t page_bytes = (size_t)(4 * ((hd + 31) / 32) + (vd / 16) * 2) * 1024;
            if (lds_bytes + 2 * page_bytes <= 144 * 1024)
                lds_bytes += 2 * page_bytes;
            else
                nc = 1;
        }
        grid = dim3((max_rows + 64 * nc - 1) / (64 * nc), n_seqs, nh);
        AGAVE_CHECK(grid.y <= 65535 && grid.z <= 65535, "attn_biased_mfma: too many sequences or heads for the grid");
    }
    if (ks > 12) {                                      // Q in LDS, behind whatever else is there
        M.q_off = (int)(lds_bytes / sizeof(float));
        lds_bytes += (size_t)(one_row ? 1 : threads / 64) * ks * 1024;
    }
    int rc = 0;
    switch (ks) {
        case 1: BIASED_VB(1); break;
        case 2: BIASED_VB(2); break;
        case 4: BIASED_VB(4); break;
        case 8: BIASED_VB(8); break;
        case 12: rc = launch_biased_mfma<12, 24>(A, M, grid, threads, nc, lds_bytes, stream); break;
        default: rc = launch_biased_mfma<18, 32>(A, M, grid, threads, nc, lds_bytes, stream); break;
    }
    if (rc) return rc;
    AGAVE_LAUNCH_CHECK("attn_biased_mfma");
    if (splits > 1) {
        attn_biased_merge_kernel<<<N * nh, vd <= 64 ? 64 : vd <= 128 ? 128 : 256, 0, stream>>>(parts, splits, nh, vd, (bf16*)out, ldo,
                                                                                      (const bf16*)gate, ldg);
        AGAVE_LAUNCH_CHECK("attn_biased_merge");
    }
    return 0;
}
