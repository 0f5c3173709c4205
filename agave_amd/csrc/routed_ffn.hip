// A routed feed-forward (mixture of experts) for gfx950: the choice of experts per token and the
// experts' products over the tokens that chose them.
//
//   s = softmax(z) over all R router outputs (32-bit);  choice score c = s + correction;
//   the R outputs form `groups` equal groups of neighbours, a group's score is its largest c, only
//   the outputs of the `keep` best groups can be chosen; the `top` largest c among them are
//   chosen (the lower index wins a tie); the weight of a chosen output is s * scale.
//   Outputs e >= E are identity experts: their result is the feed-forward's input row itself.
//   Expert e < E: W_down[e] (act(W_gate[e] x) * (W_up[e] x)).
//   The other way of scoring (mode 1): the logits z + bias decide, the `top` largest are chosen, and the weights are
//   the softmax over the chosen logits alone, times scale.
//   A third way (mode 2): s = sigmoid(z), each output on its own; choice and groups as with the softmax over all.
//   `group_top` 2: a group's score is the sum of its two largest c instead of its largest.  `normalise`: the chosen
//   outputs' weights are divided by their sum + 1e-20 before the factor.
//   The router matrix may carry further rows behind its R outputs (`extra`): their products with the token are handed
//   out as they are (the logit of a gate on the shared expert), so that they cost no kernel of their own.
//
// A (token, slot) pair p = t * top + slot names one chosen output.  The plain kernels take the pairs
// as they come (a wave per pair and output column).  The matrix-core kernels take them sorted by
// expert, in tiles of 16 or 64 pairs that never span two experts (`route_sort` makes the list and the
// tiles' table on the device, so a step's launches never depend on the choice).
#include "common_impl.h"
#include "mfma.h"
#include <math.h>

#define ROUTE_MAX 1024        // router outputs at most

// ------------------------------------------------------------------ the choice
// One thread per token; `s` [N][R] is scratch that receives the softmax.
__global__ void route_topk_kernel(const float* __restrict__ z, long ldz, const float* __restrict__ correction,
                                  float* __restrict__ s, int N, int R, int groups, int keep, int top, float scale,
                                  int* __restrict__ choice, float* __restrict__ weight) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= N) return;
    const float* zr = z + (size_t)t * ldz;
    float* sr = s + (size_t)t * R;
    float mx = -INFINITY;
    for (int e = 0; e < R; ++e) mx = fmaxf(mx, zr[e]);
    float sum = 0.f;
    for (int e = 0; e < R; ++e) {
        const float w = expf(zr[e] - mx);
        sr[e] = w;
        sum += w;
    }
    const float inv = 1.0f / sum;
    for (int e = 0; e < R; ++e) sr[e] *= inv;
    // groups that may be chosen from: a bit per group (at most 64 groups)
    const int gs = R / groups;
    unsigned long long open = ~0ull;
    if (keep < groups) {
        open = 0ull;
        for (int r = 0; r < keep; ++r) {
            int best = -1;
            float best_v = -INFINITY;
            for (int g = 0; g < groups; ++g) {
                if ((open >> g) & 1ull) continue;
                float gv = -INFINITY;
                for (int e = g * gs; e < (g + 1) * gs; ++e) gv = fmaxf(gv, sr[e] + (correction ? correction[e] : 0.f));
                if (best < 0 || gv > best_v) {
                    best = g;
                    best_v = gv;
                }
            }
            open |= 1ull << best;
        }
    }
    // the `top` best of what is open; what was chosen is marked in the scratch row's sign (s >= 0)
    for (int r = 0; r < top; ++r) {
        int best = -1;
        float best_v = -INFINITY;
        for (int e = 0; e < R; ++e) {
            const float se = sr[e];
            if (se < 0.f || !((open >> (e / gs)) & 1ull)) continue;
            const float c = se + (correction ? correction[e] : 0.f);
            if (best < 0 || c > best_v) {
                best = e;
                best_v = c;
            }
        }
        // (top <= open outputs is checked on the host, so best >= 0)
        choice[(size_t)t * top + r] = best;
        weight[(size_t)t * top + r] = sr[best] * scale;
        sr[best] = -1.0f - sr[best];
    }
}

extern "C" int agave_route_topk(const float* z, long ldz, const float* correction, float* scratch, int N, int R, int groups,
                                int keep, int top, float scale, int* choice, float* weight, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && R > 0 && R <= ROUTE_MAX, "route_topk: %d router outputs (1 to %d)", R, ROUTE_MAX);
    AGAVE_CHECK(groups > 0 && groups <= 64 && R % groups == 0, "route_topk: %d outputs in %d groups (equal groups, at most 64)", R, groups);
    AGAVE_CHECK(keep > 0 && keep <= groups, "route_topk: %d of %d groups kept", keep, groups);
    AGAVE_CHECK(top > 0 && top <= keep * (R / groups), "route_topk: %d chosen of %d that are open", top, keep * (R / groups));
    AGAVE_CHECK(z && scratch && choice && weight && ldz >= R, "route_topk: bad buffers");
    if (N == 0) return 0;
    route_topk_kernel<<<(N + 63) / 64, 64, 0, stream>>>(z, ldz, correction, scratch, N, R, groups, keep, top, scale, choice, weight);
    AGAVE_LAUNCH_CHECK("route_topk");
    return 0;
}

// ------------------------------------------------------------------ router product and choice in one kernel
// A workgroup takes RR tokens: its waves share the router's outputs (a wave per output in turn, the lanes
// along the width, a weight row read once for all of the workgroup's tokens), the logits wait in LDS, and one
// thread per token then chooses as route_topk_kernel does.  The router matrix is 32-bit; the rows may be bfloat16.
// eight neighbours along the width as floats (16 bytes of bfloat16, 32 of float)
__device__ __forceinline__ void load8(const bf16* p, float* v) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    const uint32_t r[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(r[i] << 16);
        v[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
    }
}
__device__ __forceinline__ void load8(const float* p, float* v) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

// WIDE: the width is a multiple of 8 and the rows are aligned, so a lane takes eight neighbours at a time (a
// fraction of the loads, many of them in flight); otherwise element by element.  The workgroup's waves (4, or 16
// where few tokens leave the chip idle) take the outputs in turn.
// RR tokens a workgroup: eight where there are many, one where few tokens would leave the chip idle (a wave then holds
// a whole row's share of loads in flight at once).
template <typename T, bool WIDE, int RR>
__global__ __launch_bounds__(1024) void route_rows_kernel(const T* __restrict__ x, long ldx, const float* __restrict__ router,
                                                          const float* __restrict__ correction, int N, int K, int R, int groups,
                                                          int keep, int top, float scale, int* __restrict__ choice,
                                                          float* __restrict__ weight, int mode, int extra,
                                                          float* __restrict__ extra_out, int group_top, int normalise) {
    extern __shared__ float zs[];                      // [RR][R + extra], then the corrections [R]
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int Rt = R + extra;
    float* corr = zs + RR * Rt;                // (read many times by the one thread that chooses: from LDS, not memory)
    for (int e = threadIdx.x; e < R; e += blockDim.x) corr[e] = correction ? correction[e] : 0.f;
    const int t0 = blockIdx.x * RR;
    const int rows = min(RR, N - t0);
    for (int r = w; r < Rt; r += nw) {
        const float* wr = router + (size_t)r * K;
        float acc[RR];
#pragma unroll
        for (int i = 0; i < RR; ++i) acc[i] = 0.f;
        if (WIDE) {
#pragma unroll(RR == 1 ? 4 : 2)
            for (int k = 8 * lane; k < K; k += 512) {
                float wk[8];
                load8(wr + k, wk);
#pragma unroll
                for (int i = 0; i < RR; ++i) {
                    const int t = t0 + (i < rows ? i : 0);
                    float xv[8];
                    load8(x + (size_t)t * ldx + k, xv);
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[i] = fmaf(xv[j], wk[j], acc[i]);
                }
            }
        } else {
            for (int k = lane; k < K; k += 64) {
                const float wk = wr[k];
#pragma unroll
                for (int i = 0; i < RR; ++i) {
                    const int t = t0 + (i < rows ? i : 0);
                    acc[i] = fmaf(ld(x + (size_t)t * ldx + k), wk, acc[i]);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < RR; ++i) {
            const float sum = wave_sum(acc[i]);
            if (lane == 0) zs[i * Rt + r] = sum;
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < rows * extra; i += blockDim.x)
        extra_out[(size_t)(t0 + i / extra) * extra + i % extra] = zs[(i / extra) * Rt + R + i % extra];
    // the choice: a wave per token, the lanes along the outputs
    const int gs = R / groups;
    for (int i = w; i < rows; i += nw) {
        float* sr = zs + (size_t)i * Rt;
        const int t = t0 + i;
        if (mode == 1) {
            // the largest logits (bias added) are chosen, the lower index among equals; a chosen place is marked by
            // -infinity; lane r keeps round r's logit, and the weights are the softmax over those (top <= 64)
            for (int e = lane; e < R; e += 64) sr[e] += corr[e];
            __builtin_amdgcn_wave_barrier();
            int my_choice = 0;
            float my_logit = 0.f, first_v = 0.f, sum = 0.f;
            for (int r = 0; r < top; ++r) {
                float best_v = -INFINITY;
                int best = -1;
                for (int e = lane; e < R; e += 64) {
                    const float se = sr[e];
                    if (se == -INFINITY) continue;
                    if (best < 0 || se > best_v) {
                        best = e;
                        best_v = se;
                    }
                }
                const float top_v = wave_max(best >= 0 ? best_v : -INFINITY);
                int chosen = (int)(-wave_max((best >= 0 && best_v == top_v) ? -(float)best : -INFINITY));
                if (chosen < 0 || chosen >= R) chosen = 0;          // (every open logit is -infinity or not a number)
                if (r == 0) first_v = top_v;
                sum += expf(top_v - first_v);
                if (r == lane) {
                    my_choice = chosen;
                    my_logit = top_v;
                }
                if (lane == 0) sr[chosen] = -INFINITY;
                __builtin_amdgcn_wave_barrier();
            }
            if (lane < top) {
                choice[(size_t)t * top + lane] = my_choice;
                weight[(size_t)t * top + lane] = expf(my_logit - first_v) / sum * scale;
            }
            continue;
        }
        if (mode == 2) {
            for (int e = lane; e < R; e += 64) sr[e] = 1.0f / (1.0f + expf(-sr[e]));
        } else {
            float mx = -INFINITY;
            for (int e = lane; e < R; e += 64) mx = fmaxf(mx, sr[e]);
            mx = wave_max(mx);
            float sum = 0.f;
            for (int e = lane; e < R; e += 64) {
                const float v = expf(sr[e] - mx);
                sr[e] = v;
                sum += v;
            }
            const float inv = 1.0f / wave_sum(sum);
            for (int e = lane; e < R; e += 64) sr[e] *= inv;
        }
        __builtin_amdgcn_wave_barrier();
        // the groups that stay open: lane g holds group g's score (at most 64 groups)
        unsigned long long open = ~0ull;
        if (keep < groups) {
            float gv = -INFINITY;
            if (lane < groups) {
                float second = -INFINITY;
                for (int e = lane * gs; e < (lane + 1) * gs; ++e) {
                    const float c = sr[e] + corr[e];
                    if (c > gv) {
                        second = gv;
                        gv = c;
                    } else {
                        second = fmaxf(second, c);
                    }
                }
                if (group_top == 2 && gs > 1) gv += second;
            }
            open = 0ull;
            for (int r = 0; r < keep; ++r) {
                const float cand = (lane < groups && !((open >> lane) & 1ull)) ? gv : -INFINITY;
                const float best_v = wave_max(cand);
                // the lowest group among equals
                const float first = wave_max((lane < groups && !((open >> lane) & 1ull) && cand == best_v) ? -(float)lane : -INFINITY);
                open |= 1ull << (int)(-first);
            }
        }
        // the `top` best of what is open; what was chosen is marked in the row's sign (s >= 0)
        int my_choice = 0;
        float my_weight = 0.f, chosen_sum = 0.f;
        for (int r = 0; r < top; ++r) {
            float best_v = -INFINITY;
            int best = -1;
            for (int e = lane; e < R; e += 64) {
                const float se = sr[e];
                if (se < 0.f || !((open >> (e / gs)) & 1ull)) continue;
                const float c = se + corr[e];
                if (best < 0 || c > best_v) {          // (a lane's outputs come in rising order: the first of equals stays)
                    best = e;
                    best_v = c;
                }
            }
            const float top_v = wave_max(best >= 0 ? best_v : -INFINITY);
            const int chosen = (int)(-wave_max((best >= 0 && best_v == top_v) ? -(float)best : -INFINITY));
            // (top <= open outputs is checked on the host, so some lane has a candidate)
            const float s_chosen = sr[chosen];
            chosen_sum += s_chosen;
            if ((r & 63) == lane) {             // lane r keeps round r's result; the results leave in one store at the end
                my_choice = chosen;
                my_weight = s_chosen * scale;
            }
            if (lane == 0) sr[chosen] = -1.0f - s_chosen;
            // (a wave's LDS accesses happen in the order they were issued: the next round's reads see this write)
            __builtin_amdgcn_wave_barrier();
            if ((r & 63) == 63 || r == top - 1) {
                const int at = (r & ~63) + lane;
                if (at <= r) {
                    choice[(size_t)t * top + at] = my_choice;
                    weight[(size_t)t * top + at] = normalise ? my_weight / (chosen_sum + 1e-20f) : my_weight;      // (normalise: top <= 64, one batch)
                }
            }
        }
    }
}

extern "C" int agave_route_rows(int dtype, const void* x, long ldx, const float* router, const float* correction, int N, int K,
                                int R, int groups, int keep, int top, float scale, int* choice, float* weight, int mode,
                                int extra, float* extra_out, int group_top, int normalise, hipStream_t stream) {
    AGAVE_CHECK(mode == 0 || mode == 2 || (mode == 1 && top <= 64 && groups == 1), "route_rows: the softmax over the chosen logits takes at most 64 of them and no groups");
    AGAVE_CHECK((group_top == 1 || group_top == 2) && (!normalise || (top <= 64 && mode != 1)), "route_rows: a group counts by its largest or its two largest; weights are divided by their sum for at most 64 chosen");
    AGAVE_CHECK(extra >= 0 && extra <= 64 && (extra == 0 || extra_out), "route_rows: %d further rows of the router (0 to 64, with a place for their products)", extra);
    AGAVE_CHECK(N >= 0 && K > 0 && R > 0 && R <= ROUTE_MAX, "route_rows: %d router outputs (1 to %d)", R, ROUTE_MAX);
    AGAVE_CHECK(groups > 0 && groups <= 64 && R % groups == 0, "route_rows: %d outputs in %d groups (equal groups, at most 64)", R, groups);
    AGAVE_CHECK(keep > 0 && keep <= groups, "route_rows: %d of %d groups kept", keep, groups);
    AGAVE_CHECK(top > 0 && top <= keep * (R / groups), "route_rows: %d chosen of %d that are open", top, keep * (R / groups));
    AGAVE_CHECK(x && router && choice && weight && ldx >= K, "route_rows: bad buffers");
    if (N == 0) return 0;
    const bool wide = K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 32) == 0 && ((uintptr_t)router % 32) == 0;
    AGAVE_CHECK(dtype == AGAVE_F32 || dtype == AGAVE_BF16, "route_rows: unknown dtype %d", dtype);
    const bool f32 = dtype == AGAVE_F32;
    if (N <= 64) {
        const size_t lds = (size_t)(2 * R + extra) * sizeof(float);
#define ROUTE_GO(T_, W_) route_rows_kernel<T_, W_, 1><<<N, 1024, lds, stream>>>((const T_*)x, ldx, router, correction, N, K, R, groups, keep, top, scale, choice, weight, mode, extra, extra_out, group_top, normalise)
        if (f32 && wide) ROUTE_GO(float, true); else if (f32) ROUTE_GO(float, false); else if (wide) ROUTE_GO(bf16, true); else ROUTE_GO(bf16, false);
#undef ROUTE_GO
    } else {
        const int blocks = (N + 7) / 8;
        const size_t lds = (size_t)(9 * R + 8 * extra) * sizeof(float);
        const int threads = blocks <= 512 ? 1024 : 256;        // (more waves to share the outputs while they all fit the chip at once)
#define ROUTE_GO(T_, W_) route_rows_kernel<T_, W_, 8><<<blocks, threads, lds, stream>>>((const T_*)x, ldx, router, correction, N, K, R, groups, keep, top, scale, choice, weight, mode, extra, extra_out, group_top, normalise)
        if (f32 && wide) ROUTE_GO(float, true); else if (f32) ROUTE_GO(float, false); else if (wide) ROUTE_GO(bf16, true); else ROUTE_GO(bf16, false);
#undef ROUTE_GO
    }
    AGAVE_LAUNCH_CHECK("route_rows");
    return 0;
}

// ------------------------------------------------------------------ activations of the experts' gates
// act(gate) * up for activations 0 to 3; 6 ("swish_clamped"): g = min(gate, p0), u = clamp(up, -p0, p0),
// g sigmoid(p1 g) (u + 1)
__device__ __forceinline__ float expert_act(float x, int act);
__device__ __forceinline__ float expert_gated(float gate, float up, int act, float p0, float p1) {
    if (act == 6) {
        const float g = fminf(gate, p0), u = fminf(fmaxf(up, -p0), p0);
        return g / (1.0f + expf(-p1 * g)) * (u + 1.0f);
    }
    return expert_act(gate, act) * up;
}
__device__ __forceinline__ float expert_act(float x, int act) {
    switch (act) {
        case 0: { const float c = 0.7978845608028654f; return 0.5f * x * (1.0f + tanhf(c * (x + 0.044715f * x * x * x))); }
        case 1: return x / (1.0f + expf(-x));
        case 2: return 0.5f * x * (1.0f + erff(x * 0.7071067811865476f));
        default: return x > 0.f ? x : 0.f;
    }
}

// ------------------------------------------------------------------ plain products, pair by pair
// act[p][f] = act(W_gate[e] x_t . f) * (W_up[e] x_t . f): a wave per (pair, f), lanes along K
template <typename T>
__global__ __launch_bounds__(256) void routed_gate_up_plain_kernel(const T* __restrict__ x, long ldx, const int* __restrict__ choice,
                                                                   const T* __restrict__ wg, const T* __restrict__ wu,
                                                                   T* __restrict__ act_out, int top, int E, int ff, int K, int act,
                                                                   float p0, float p1) {
    const int p = blockIdx.x;
    const int e = choice[p];
    if (e < 0 || e >= E) return;
    const int lane = threadIdx.x & 63;
    const int f = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (f >= ff) return;
    const T* xr = x + (size_t)(p / top) * ldx;
    const T* g = wg + ((size_t)e * ff + f) * K;
    const T* u = wu + ((size_t)e * ff + f) * K;
    float ag = 0.f, au = 0.f;
    for (int k = lane; k < K; k += 64) {
        const float xv = ld(xr + k);
        ag = fmaf(xv, ld(g + k), ag);
        au = fmaf(xv, ld(u + k), au);
    }
    ag = wave_sum(ag);
    au = wave_sum(au);
    // (the gate's sum is rounded to the rows' element type before the activation, as a product that
    // writes its rows and an activation kernel that reads them would)
    if (lane == 0) {
        T tg, tu;
        st(&tg, ag);
        st(&tu, au);
        st(act_out + (size_t)p * ff + f, expert_gated(ld(&tg), ld(&tu), act, p0, p1));
    }
}

// y[p][c] = W_down[e][c] . act[p]: a wave per (pair, c), lanes along ff; y is 32-bit
template <typename T>
__global__ __launch_bounds__(256) void routed_down_plain_kernel(const T* __restrict__ act_in, const int* __restrict__ choice,
                                                                const T* __restrict__ wd, float* __restrict__ y, int E, int ff,
                                                                int hidden) {
    const int p = blockIdx.x;
    const int e = choice[p];
    if (e < 0 || e >= E) return;
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (c >= hidden) return;
    const T* a = act_in + (size_t)p * ff;
    const T* w = wd + ((size_t)e * hidden + c) * ff;
    float acc = 0.f;
    for (int f = lane; f < ff; f += 64) acc = fmaf(ld(a + f), ld(w + f), acc);
    acc = wave_sum(acc);
    if (lane == 0) y[(size_t)p * hidden + c] = acc;
}

// out[t] = sum over the token's pairs of weight * (expert row, or the input row for an identity expert) + shared[t].
// `place` (may be null): where pair p's row lies in y (a sorted list); null: at p.
template <typename T>
__global__ void routed_combine_kernel(const float* __restrict__ y, const int* __restrict__ place, const int* __restrict__ choice,
                                      const float* __restrict__ weight, const T* __restrict__ x, long ldx,
                                      const T* __restrict__ shared, long lds, const float* __restrict__ shared_gate,
                                      T* __restrict__ out, long ldo, int N, int top, int E, int hidden) {
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)N * hidden) return;
    const int t = (int)(idx / hidden), c = (int)(idx % hidden);
    // (no load under a per-lane condition: the input row's element is read once, an expert row's from a row that exists
    // whatever the choice, and what does not count is left out afterwards)
    const float xv = ld(x + (size_t)t * ldx + c);
    const float sv = ld((shared ? shared : x) + (size_t)t * (shared ? lds : ldx) + c);
    float acc = 0.f;
#pragma unroll 4
    for (int r = 0; r < top; ++r) {
        const int p = t * top + r;
        const int e = choice[p];
        const float w = weight[p];
        const bool expert = e >= 0 && e < E;
        int row = place ? place[p] : p;
        row = (expert && row >= 0) ? row : 0;
        const float yv = y ? y[(size_t)row * hidden + c] : 0.f;
        acc = fmaf(w, e >= E ? xv : (expert ? yv : 0.f), acc);
    }
    // (the shared expert's row, times the sigmoid of a logit per token where it has a gate)
    if (shared) acc = shared_gate ? fmaf(1.0f / (1.0f + expf(-shared_gate[t])), sv, acc) : acc + sv;
    st(out + (size_t)t * ldo + c, acc);
}

extern "C" int agave_routed_experts_plain(int dtype, const void* x, long ldx, const int* choice, const void* wg, const void* wu,
                                          const void* wd, void* act_rows, float* y, int N, int top, int E, int ff, int hidden,
                                          int act, float p0, float p1, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && top > 0 && E >= 0 && ff > 0 && hidden > 0, "routed_experts: bad sizes");
    AGAVE_CHECK((act >= 0 && act < 4) || act == 6, "routed_experts: unknown activation %d", act);
    AGAVE_CHECK(x && choice && act_rows && y && ldx >= hidden && (E == 0 || (wg && wu && wd)), "routed_experts: bad buffers");
    AGAVE_CHECK((ff + 3) / 4 <= 65535 && (hidden + 3) / 4 <= 65535, "routed_experts: too many columns for the grid");
    if (N == 0 || E == 0) return 0;
    const dim3 g1(N * top, (ff + 3) / 4), g2(N * top, (hidden + 3) / 4);
    if (dtype == AGAVE_F32) {
        routed_gate_up_plain_kernel<float><<<g1, 256, 0, stream>>>((const float*)x, ldx, choice, (const float*)wg, (const float*)wu,
                                                                   (float*)act_rows, top, E, ff, hidden, act, p0, p1);
        routed_down_plain_kernel<float><<<g2, 256, 0, stream>>>((const float*)act_rows, choice, (const float*)wd, y, E, ff, hidden);
    } else if (dtype == AGAVE_BF16) {
        routed_gate_up_plain_kernel<bf16><<<g1, 256, 0, stream>>>((const bf16*)x, ldx, choice, (const bf16*)wg, (const bf16*)wu,
                                                                  (bf16*)act_rows, top, E, ff, hidden, act, p0, p1);
        routed_down_plain_kernel<bf16><<<g2, 256, 0, stream>>>((const bf16*)act_rows, choice, (const bf16*)wd, y, E, ff, hidden);
    } else
        AGAVE_CHECK(false, "routed_experts: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("routed_experts_plain");
    return 0;
}

extern "C" int agave_routed_combine(int dtype, const float* y, const int* place, const int* choice, const float* weight,
                                    const void* x, long ldx, const void* shared, long lds, const float* shared_gate, void* out,
                                    long ldo, int N, int top, int E, int hidden, hipStream_t stream) {
    AGAVE_CHECK(N >= 0 && top > 0 && hidden > 0, "routed_combine: bad sizes");
    AGAVE_CHECK(choice && weight && x && out && (E == 0 || y) && ldx >= hidden && ldo >= hidden && (!shared || lds >= hidden),
                "routed_combine: bad buffers");
    if (N == 0) return 0;
    const long total = (long)N * hidden;
    const int blocks = (int)((total + 255) / 256);
    if (dtype == AGAVE_F32)
        routed_combine_kernel<float><<<blocks, 256, 0, stream>>>(y, place, choice, weight, (const float*)x, ldx, (const float*)shared,
                                                                 lds, shared_gate, (float*)out, ldo, N, top, E, hidden);
    else if (dtype == AGAVE_BF16)
        routed_combine_kernel<bf16><<<blocks, 256, 0, stream>>>(y, place, choice, weight, (const bf16*)x, ldx, (const bf16*)shared,
                                                                lds, shared_gate, (bf16*)out, ldo, N, top, E, hidden);
    else
        AGAVE_CHECK(false, "routed_combine: unknown dtype %d", dtype);
    AGAVE_LAUNCH_CHECK("routed_combine");
    return 0;
}

// ------------------------------------------------------------------ the pairs sorted by expert
// One workgroup.  Every expert's pairs get a run of whole tiles of TM sorted rows (the last one padded):
//   place[p]        sorted row of pair p (-1: the pair's choice is an identity expert)
//   sorted_pair[r]  pair in sorted row r (-1: padding)
//   tile_expert[t]  expert of tile t (-1: no such tile)
// The order of an expert's pairs among themselves is whatever the atomics make it; every row's result is
// its own, so nothing depends on it.
__global__ __launch_bounds__(1024) void route_sort_kernel(const int* __restrict__ choice, int P, int E, int TM, int cap,
                                                          int max_tiles, int* __restrict__ place,
                                                          int* __restrict__ sorted_pair, int* __restrict__ tile_expert) {
    __shared__ int counts[ROUTE_MAX];
    __shared__ int first_row[ROUTE_MAX];
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += blockDim.x) counts[e] = 0;
    for (int r = tid; r < cap; r += blockDim.x) sorted_pair[r] = -1;
    for (int t = tid; t < max_tiles; t += blockDim.x) tile_expert[t] = -1;
    __syncthreads();
    for (int p = tid; p < P; p += blockDim.x) {
        const int e = choice[p];
        place[p] = (e >= 0 && e < E) ? atomicAdd(&counts[e], 1) : -1;        // for now: the pair's rank within its expert
    }
    __syncthreads();
    if (tid == 0) {
        int tile = 0;
        for (int e = 0; e < E; ++e) {
            first_row[e] = tile * TM;
            const int n = (counts[e] + TM - 1) / TM;
            for (int i = 0; i < n && tile + i < max_tiles; ++i) tile_expert[tile + i] = e;
            tile += n;
        }
    }
    __syncthreads();
    for (int p = tid; p < P; p += blockDim.x) {
        const int e = choice[p];
        if (e >= 0 && e < E) {
            const int r = first_row[e] + place[p];
            if (r < cap) {
                place[p] = r;
                sorted_pair[r] = p;
            } else {
                place[p] = -1;          // (cannot happen: cap holds every pair and every expert's padding)
            }
        }
    }
}

extern "C" int agave_route_sort(const int* choice, int P, int E, int TM, int cap, int max_tiles, int* place, int* sorted_pair,
                                int* tile_expert, hipStream_t stream) {
    AGAVE_CHECK(P >= 0 && E > 0 && E <= ROUTE_MAX && (TM == 16 || TM == 64), "route_sort: bad sizes P=%d E=%d TM=%d", P, E, TM);
    AGAVE_CHECK(max_tiles >= (P + TM - 1) / TM + E && cap >= max_tiles * TM, "route_sort: %d tiles of %d rows do not hold %d pairs of %d experts",
                max_tiles, TM, P, E);
    AGAVE_CHECK(choice && place && sorted_pair && tile_expert, "route_sort: null buffer");
    if (P == 0) return 0;
    route_sort_kernel<<<1, 1024, 0, stream>>>(choice, P, E, TM, cap, max_tiles, place, sorted_pair, tile_expert);
    AGAVE_LAUNCH_CHECK("route_sort");
    return 0;
}

// ------------------------------------------------------------------ the experts' products on the matrix cores
// A workgroup takes one tile of TM = 16 MI sorted rows (one expert) and 64 NJ output columns, 16 NJ a wave; both operands
// come straight from memory in the order v_mfma_f32_16x16x32_bf16 reads them (a lane's eight neighbours along K are
// 16 bytes of a row of X or of W[e]).  GATED: two products (gate and up) side by side, ending in act(gate) * up,
// rows gathered from X through the sorted pairs; otherwise one product of the sorted inner rows, 32-bit out.
template <int MI, int NJ, bool GATED>
__global__ __launch_bounds__(256) void routed_product_mfma_kernel(const bf16* __restrict__ x, long ldx, const int* __restrict__ sorted_pair,
                                                                  const int* __restrict__ tile_expert, const bf16* __restrict__ w0,
                                                                  const bf16* __restrict__ w1, void* __restrict__ out_, int top,
                                                                  int n_out, int K, int act, int wpacked, float p0, float p1) {
    const int e = tile_expert[blockIdx.x];
    if (e < 0) return;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int row0 = blockIdx.x * 16 * MI;
    // A tile of 16 rows (MI == 1) streams its weights once: its four waves take the same 16 NJ columns and a quarter of
    // K each, so that a wave's chain of loads is a quarter as long, and wave 0 adds the four sums through LDS.
    constexpr bool KSPLIT = MI == 1;
    const int col0 = KSPLIT ? blockIdx.y * (16 * NJ) : blockIdx.y * (64 * NJ) + w * (16 * NJ);
    if (col0 >= n_out) return;                                  // (the whole workgroup where the waves split K)
    const int k_share = KSPLIT ? ((K + 127) / 128) * 32 : K;    // whole steps of 32
    const int k_begin = KSPLIT ? min(K, w * k_share) : 0, k_end = KSPLIT ? min(K, k_begin + k_share) : K;
    // A rows: 16 i + c of the tile
    const bf16* arow[MI];
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int r = row0 + 16 * i + c;
        if (GATED) {
            const int p = sorted_pair[r];
            arow[i] = x + (size_t)(p >= 0 ? p / top : 0) * ldx + 8 * g;       // (a padding row computes on row 0 and is never read)
        } else {
            arow[i] = x + (size_t)r * ldx + 8 * g;
        }
    }
    // B rows: output columns col0 + 16 j + c of expert e (clamped; columns past the end are not stored)
    const bf16* b0[NJ];
    const bf16* b1[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        int col = col0 + 16 * j + c;
        if (col >= n_out) col = n_out - 1;
        // (wpacked: W[e] in tiles of 16 rows x 32 columns, each the 64 lanes' operands in a row, a row block's tiles one
        // after another: a whole operand is one load of a kilobyte)
        const size_t at0 = wpacked ? (((size_t)e * (n_out / 16) + col / 16) * (K / 32) * 64 + lane) * 8
                                   : ((size_t)e * n_out + col) * K + 8 * g;
        b0[j] = w0 + at0;
        b1[j] = GATED ? w1 + at0 : nullptr;
    }
    f32x4_t acc0[MI][NJ], acc1[MI][GATED ? NJ : 1];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            acc0[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            if (GATED) acc1[i][GATED ? j : 0] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
    int k_done = k_begin;
    if constexpr (MI == 1) {
        // a tile of 16 rows streams its weights once and waits for memory, not for the matrix cores: the loads of
        // eight steps are asked for before the first is used
        constexpr int U = 8;
        for (; k_done + 32 * U <= k_end; k_done += 32 * U) {
            frag16 a[U], bw0[U][NJ], bw1[U][NJ];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int k0 = k_done + 32 * u;
                a[u].u = *reinterpret_cast<const uint4*>(arow[0] + k0);
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    bw0[u][j].u = *reinterpret_cast<const uint4*>(b0[j] + (wpacked ? k0 * 16 : k0));
                    if (GATED) bw1[u][j].u = *reinterpret_cast<const uint4*>(b1[j] + (wpacked ? k0 * 16 : k0));
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    acc0[0][j] = mfma_16x16x32(a[u], bw0[u][j], acc0[0][j]);
                    if (GATED) acc1[0][GATED ? j : 0] = mfma_16x16x32(a[u], bw1[u][j], acc1[0][GATED ? j : 0]);
                }
        }
    }
    for (int k0 = k_done; k0 < k_end; k0 += 32) {
        // (loads without conditions, from inside the row; a lane past the row's end reads its start and is emptied)
        const bool in = k0 + 8 * g < K;
        const int at = in ? k0 : -8 * g;
        const int bat = wpacked ? k0 * 16 : at;
        frag16 a[MI], bw0[NJ], bw1[NJ];
#pragma unroll
        for (int i = 0; i < MI; ++i) a[i].u = *reinterpret_cast<const uint4*>(arow[i] + at);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            bw0[j].u = *reinterpret_cast<const uint4*>(b0[j] + bat);
            if (GATED) bw1[j].u = *reinterpret_cast<const uint4*>(b1[j] + bat);
        }
        if (!in) {
#pragma unroll
            for (int i = 0; i < MI; ++i) a[i].u = make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                acc0[i][j] = mfma_16x16x32(a[i], bw0[j], acc0[i][j]);
                if (GATED) acc1[i][GATED ? j : 0] = mfma_16x16x32(a[i], bw1[j], acc1[i][GATED ? j : 0]);
            }
    }
    if constexpr (KSPLIT) {
        __shared__ float part[3][2][NJ][256];
        if (w > 0) {
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    part[w - 1][0][j][e4 * 64 + lane] = acc0[0][j][e4];
                    if (GATED) part[w - 1][1][j][e4 * 64 + lane] = acc1[0][GATED ? j : 0][e4];
                }
        }
        __syncthreads();
        if (w > 0) return;
#pragma unroll
        for (int ow = 0; ow < 3; ++ow)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    acc0[0][j][e4] += part[ow][0][j][e4 * 64 + lane];
                    if (GATED) acc1[0][GATED ? j : 0][e4] += part[ow][1][j][e4 * 64 + lane];
                }
    }
    // D[i][j]: lane holds rows 4 g + e4 of the row block, column c of the column block
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int col = col0 + 16 * j + c;
            if (col >= n_out) continue;
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const size_t r = (size_t)row0 + 16 * i + 4 * g + e4;
                if (GATED) {
                    // (gate and up are rounded to the rows' type before the activation, as the plain kernel does)
                    const float gt = bf16_to_f32(f32_to_bf16(acc0[i][j][e4])), up = bf16_to_f32(f32_to_bf16(acc1[i][GATED ? j : 0][e4]));
                    ((bf16*)out_)[r * n_out + col] = f32_to_bf16(expert_gated(gt, up, act, p0, p1));
                } else {
                    ((float*)out_)[r * n_out + col] = acc0[i][j][e4];
                }
            }
        }
}

// act_rows [cap, ff] bfloat16 and y [cap, hidden] float32 hold sorted rows (see route_sort)
extern "C" int agave_routed_experts_mfma(const void* x, long ldx, const int* sorted_pair, const int* tile_expert, const void* wg,
                                         const void* wu, const void* wd, void* act_rows, float* y, int TM, int max_tiles, int top,
                                         int E, int ff, int hidden, int act, int wpacked, float p0, float p1, hipStream_t stream) {
    AGAVE_CHECK(!wpacked || (ff % 32 == 0 && hidden % 32 == 0), "routed_experts_mfma: weights in tile order need sizes that are multiples of 32");
    AGAVE_CHECK(max_tiles > 0 && top > 0 && E > 0 && ff > 0 && hidden > 0 && (TM == 16 || TM == 64), "routed_experts_mfma: bad sizes");
    AGAVE_CHECK((act >= 0 && act < 4) || act == 6, "routed_experts_mfma: unknown activation %d", act);
    AGAVE_CHECK(hidden % 8 == 0 && ff % 8 == 0 && ldx % 8 == 0, "routed_experts_mfma: sizes must be multiples of 8 (hidden %d, ff %d)", hidden, ff);
    AGAVE_CHECK(x && sorted_pair && tile_expert && wg && wu && wd && act_rows && y, "routed_experts_mfma: null buffer");
    AGAVE_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)wg % 16) == 0 && ((uintptr_t)wu % 16) == 0 && ((uintptr_t)wd % 16) == 0 &&
                ((uintptr_t)act_rows % 16) == 0, "routed_experts_mfma: buffers must be aligned to 16 bytes");
    // tiles of 64 rows take 64 columns a wave (an operand that was loaded serves more multiplications); a tile of
    // 16 rows, which streams its weights once, takes 16 columns a workgroup, whose waves share K
    const int cols = TM == 64 ? 256 : 16;
    const dim3 g1(max_tiles, (ff + cols - 1) / cols), g2(max_tiles, (hidden + cols - 1) / cols);
    AGAVE_CHECK(g1.y <= 65535 && g2.y <= 65535, "routed_experts_mfma: too many columns for the grid");
    if (TM == 64) {
        routed_product_mfma_kernel<4, 4, true><<<g1, 256, 0, stream>>>((const bf16*)x, ldx, sorted_pair, tile_expert, (const bf16*)wg,
                                                                    (const bf16*)wu, act_rows, top, ff, hidden, act, wpacked, p0, p1);
        routed_product_mfma_kernel<4, 4, false><<<g2, 256, 0, stream>>>((const bf16*)act_rows, ff, sorted_pair, tile_expert, (const bf16*)wd,
                                                                     nullptr, y, top, hidden, ff, act, wpacked, p0, p1);
    } else {
        routed_product_mfma_kernel<1, 1, true><<<g1, 256, 0, stream>>>((const bf16*)x, ldx, sorted_pair, tile_expert, (const bf16*)wg,
                                                                    (const bf16*)wu, act_rows, top, ff, hidden, act, wpacked, p0, p1);
        routed_product_mfma_kernel<1, 1, false><<<g2, 256, 0, stream>>>((const bf16*)act_rows, ff, sorted_pair, tile_expert, (const bf16*)wd,
                                                                     nullptr, y, top, hidden, ff, act, wpacked, p0, p1);
    }
    AGAVE_LAUNCH_CHECK("routed_experts_mfma");
    return 0;
}
