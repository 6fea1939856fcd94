// A feed-forward of routed experts: every token goes through the `top` experts with the largest router
// scores and takes their outputs weighted by the softmax over those scores only.  An expert is
// W_d (silu(W_g h) * (W_u h)) without biases; the experts' matrices lie stacked, [E][2 F][W] for gate (an expert's
// first F rows) and up (its last F) and [E][W][F] for down.
//
//   route:  scores (the router product's float sums) + bias -> the chosen experts and their shares, float;
//           ties go to the lower expert number.
//   up:     y[t, s, :] = silu(W_g[e] h_t) * (W_u[e] h_t) for slot s of token t with e its expert.
//   down:   x[t, :] += sum_s share[t, s] * W_d[e_s] y[t, s, :], slots added in slot order in float.
// `up` and `down` read an expert's rows once per (token, slot): the form for steps of few tokens, where the
// experts' weights are what a step reads.  Steps of many tokens go expert by expert through the library's matrix
// products instead: `sort` groups the (token, slot) pairs by expert, `gather` copies their rows into that order,
// and `combine` adds every token's weighted outputs back in slot order.
#include "common.h"

#define RX_MAX_PER_LANE 8          // experts a lane keeps: up to 512 experts

// grid (T), one wave a token.
__global__ __launch_bounds__(64) void route_topk_kernel(const float* __restrict__ scores, const float* __restrict__ bias,
                                                        int* __restrict__ chosen, float* __restrict__ share, int E, int top, float out_scale) {
    const int t = blockIdx.x, lane = threadIdx.x;
    float z[RX_MAX_PER_LANE];
#pragma unroll
    for (int i = 0; i < RX_MAX_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        z[i] = e < E ? scores[(size_t)t * E + e] + (bias ? bias[e] : 0.f) : -INFINITY;
    }
    float first = 0.f, total = 0.f, mine = 0.f;
    for (int s = 0; s < top; ++s) {
        float best = -INFINITY;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < RX_MAX_PER_LANE; ++i) {
            const int e = lane + 64 * i;
            if (e < E && (z[i] > best || (z[i] == best && e < at))) { best = z[i]; at = e; }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, WAVE);
            const int oa = __shfl_xor(at, o, WAVE);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
        if (at >= E) { at = s; best = first; }    // scores that compare with nothing (a padding row's): any expert will do
        if (s == 0) first = best;                 // the largest score: the softmax's shift
        const float w = expf(best - first);
        total += w;
        if (lane == s) mine = w;                  // lane s keeps slot s's weight
        if (lane == 0) chosen[(size_t)t * top + s] = at;
#pragma unroll
        for (int i = 0; i < RX_MAX_PER_LANE; ++i)
            if (lane + 64 * i == at) z[i] = -INFINITY;
    }
    if (lane < top) share[(size_t)t * top + lane] = mine / total * out_scale;
}

extern "C" int br_route_topk(const float* scores, const float* bias, int* chosen, float* share, int T, int E, int top,
                             float out_scale, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (E <= 0 || E > 64 * RX_MAX_PER_LANE || top <= 0 || top > E || top > 64) return BR_BAD_ARG;
    route_topk_kernel<<<T, 64, 0, s>>>(scores, bias, chosen, share, E, top, out_scale);
    return br_check_launch();
}

// Routing by sigmoid scores with a choice correction and groups of experts.  s = sigmoid(z); the choice is made on
// c = s + correction, the shares on s.  With `groups` > 1 the experts form that many runs of E / groups neighbours; a
// run's score is the sum of its two largest c (of its one, where a run is one expert), only experts of the `keep`
// best runs can be chosen (the others count as minus infinity), ties to the lower number everywhere.  The shares are
// the chosen experts' s over their sum (+ 1e-20), times `out_scale`.  grid (T), one wave a token.
// Nothing is found by rounds of wave-wide maxima: every expert counts the experts that go before it (a larger c, or
// the same c and a lower number) by reading all c from LDS, and is chosen when fewer than `top` do, its count being
// its place among the chosen; the runs are kept the same way.  LDS: E + groups + 128 words.
// NPL: experts (and runs) a lane holds; the launcher takes this kernel up to 64 experts (NPL 1).
template <int NPL>
__global__ __launch_bounds__(64) void route_sigmoid_kernel(const float* __restrict__ scores, const float* __restrict__ correction,
                                                           int* __restrict__ chosen, float* __restrict__ share, int E, int top,
                                                           int groups, int keep, float out_scale) {
    extern __shared__ float rs_lds[];
    float* cs = rs_lds;                     // [E] the choice scores
    float* gsL = cs + E;                    // [groups] the runs' scores, then whether a run is kept
    float* picked = gsL + groups;           // [64] the chosen experts' s by their place
    int* who = (int*)(picked + 64);         // [64] the chosen experts by their place
    const int t = blockIdx.x, lane = threadIdx.x;
    float sg[NPL], z[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const int e = lane + 64 * i;
        sg[i] = 0.f;
        z[i] = -INFINITY;
        if (e < E) {
            sg[i] = 1.0f / (1.0f + expf(-scores[(size_t)t * E + e]));
            z[i] = sg[i] + (correction ? correction[e] : 0.f);
            cs[e] = z[i];
        }
    }
    // a place for every slot whatever the scores are (a padding row's may compare with nothing)
    if (lane < top) { who[lane] = lane; picked[lane] = 0.f; }
    __syncthreads();
    if (groups > 1) {
        const int per = E / groups;
        float gs[NPL];
#pragma unroll
        for (int j = 0; j < NPL; ++j) {
            const int g = lane + 64 * j;
            gs[j] = -INFINITY;
            if (g < groups) {
                float b1 = -INFINITY, b2 = -INFINITY;
                for (int i = 0; i < per; ++i) {
                    const float v = cs[g * per + i];
                    if (v > b1) { b2 = b1; b1 = v; } else if (v > b2) b2 = v;
                }
                gs[j] = per > 1 ? b1 + b2 : b1;
                gsL[g] = gs[j];
            }
        }
        __syncthreads();
        int before[NPL];
#pragma unroll
        for (int j = 0; j < NPL; ++j) before[j] = 0;
#pragma unroll 8
        for (int h = 0; h < groups; ++h) {
            const float o = gsL[h];
#pragma unroll
            for (int j = 0; j < NPL; ++j) before[j] += (o > gs[j] || (o == gs[j] && h < lane + 64 * j)) ? 1 : 0;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NPL; ++j) {
            const int g = lane + 64 * j;
            if (g < groups) gsL[g] = before[j] < keep ? 1.f : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NPL; ++i) {
            const int e = lane + 64 * i;
            if (e < E && gsL[e / per] == 0.f) { z[i] = -INFINITY; cs[e] = -INFINITY; }
        }
        __syncthreads();
    }
    int place[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) place[i] = 0;
#pragma unroll 8
    for (int j = 0; j < E; ++j) {              // eight reads on their way at a time
        const float o = cs[j];
#pragma unroll
        for (int i = 0; i < NPL; ++i) place[i] += (o > z[i] || (o == z[i] && j < lane + 64 * i)) ? 1 : 0;
    }
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const int e = lane + 64 * i;
        if (e < E && place[i] < top) {
            who[place[i]] = e;
            picked[place[i]] = sg[i];
        }
    }
    __syncthreads();
    if (lane < top) {
        float total = 0.f;
        for (int s = 0; s < top; ++s) total += picked[s];          // in the order of the places
        share[(size_t)t * top + lane] = picked[lane] / (total + 1e-20f) * out_scale;
        chosen[(size_t)t * top + lane] = who[lane];
    }
}

// The same for more than 64 experts, where a lane holds several: the kept runs and then the `top` experts are taken one
// after the other by rounds of wave-wide maxima (counting places would walk every choice score once per expert a lane
// holds: 51 us at 256 experts against 9).  LDS: E floats.
__global__ __launch_bounds__(64) void route_sigmoid_rounds_kernel(const float* __restrict__ scores, const float* __restrict__ correction,
                                                           int* __restrict__ chosen, float* __restrict__ share, int E, int top,
                                                           int groups, int keep, float out_scale) {
    extern __shared__ float cs[];           // the choice scores
    const int t = blockIdx.x, lane = threadIdx.x;
    float sg[RX_MAX_PER_LANE], z[RX_MAX_PER_LANE];
#pragma unroll
    for (int i = 0; i < RX_MAX_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        sg[i] = 0.f;
        z[i] = -INFINITY;
        if (e < E) {
            sg[i] = 1.0f / (1.0f + expf(-scores[(size_t)t * E + e]));
            z[i] = sg[i] + (correction ? correction[e] : 0.f);
            cs[e] = z[i];
        }
    }
    if (groups > 1) {
        __syncthreads();
        const int per = E / groups;
        // lane g scores run g + 64 j; the best `keep` runs are taken one after the other
        float gs[RX_MAX_PER_LANE];
#pragma unroll
        for (int j = 0; j < RX_MAX_PER_LANE; ++j) {
            const int g = lane + 64 * j;
            gs[j] = -INFINITY;
            if (g < groups) {
                float b1 = -INFINITY, b2 = -INFINITY;
                for (int i = 0; i < per; ++i) {
                    const float v = cs[g * per + i];
                    if (v > b1) { b2 = b1; b1 = v; } else if (v > b2) b2 = v;
                }
                gs[j] = per > 1 ? b1 + b2 : b1;
            }
        }
        __syncthreads();
        for (int e = lane; e < E; e += 64) cs[e] = -INFINITY;      // now: minus infinity unless the expert's run is kept
        __syncthreads();
        for (int r = 0; r < keep; ++r) {
            float best = -INFINITY;
            int at = 0x7fffffff;
#pragma unroll
            for (int j = 0; j < RX_MAX_PER_LANE; ++j) {
                const int g = lane + 64 * j;
                if (g < groups && gs[j] != -INFINITY && (gs[j] > best || (gs[j] == best && g < at)) ) { best = gs[j]; at = g; }
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const float ob = __shfl_xor(best, o, WAVE);
                const int oa = __shfl_xor(at, o, WAVE);
                if (oa < 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
            }
            if (at == 0x7fffffff) break;          // fewer runs with a score than `keep`
#pragma unroll
            for (int j = 0; j < RX_MAX_PER_LANE; ++j)
                if (lane + 64 * j == at) gs[j] = -INFINITY;
            for (int i = lane; i < per; i += 64) cs[at * per + i] = 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < RX_MAX_PER_LANE; ++i) {
            const int e = lane + 64 * i;
            if (e < E && cs[e] != 0.f) z[i] = -INFINITY;
        }
    }
    float total = 0.f, mine = 0.f;
    for (int s = 0; s < top; ++s) {
        float best = -INFINITY, bs = 0.f;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < RX_MAX_PER_LANE; ++i) {
            const int e = lane + 64 * i;
            if (e < E && (z[i] > best || (z[i] == best && e < at))) { best = z[i]; at = e; bs = sg[i]; }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, WAVE), os = __shfl_xor(bs, o, WAVE);
            const int oa = __shfl_xor(at, o, WAVE);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; bs = os; }
        }
        if (at >= E) { at = s; bs = 0.f; }        // scores that compare with nothing (a padding row's): any expert will do
        total += bs;
        if (lane == s) mine = bs;                 // lane s keeps slot s's score
        if (lane == 0) chosen[(size_t)t * top + s] = at;
#pragma unroll
        for (int i = 0; i < RX_MAX_PER_LANE; ++i)
            if (lane + 64 * i == at) z[i] = -INFINITY;
    }
    if (lane < top) share[(size_t)t * top + lane] = mine / (total + 1e-20f) * out_scale;
}

extern "C" int br_route_sigmoid(const float* scores, const float* correction, int* chosen, float* share, int T, int E, int top,
                                int groups, int keep, float out_scale, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (E <= 0 || E > 64 * RX_MAX_PER_LANE || top <= 0 || top > E || top > 64 || groups <= 0 || E % groups ||
        (groups > 1 && (keep <= 0 || keep > groups)))
        return BR_BAD_ARG;
    const size_t lds = (size_t)(E + groups + 128) * sizeof(float);
    if (E <= 64) route_sigmoid_kernel<1><<<T, 64, lds, s>>>(scores, correction, chosen, share, E, top, groups, keep, out_scale);
    else route_sigmoid_rounds_kernel<<<T, 64, (size_t)E * sizeof(float), s>>>(scores, correction, chosen, share, E, top, groups, keep, out_scale);
    return br_check_launch();
}

template <typename T> struct rx_vec;
template <> struct rx_vec<float> { static constexpr int N = 4; typedef f32x4 type; };
template <> struct rx_vec<bf16> { static constexpr int N = 8; typedef bf16x8 type; };

// One weight row times the activations in LDS (float), lanes across k; VEC: 16-byte loads.
template <typename T, bool VEC>
__device__ __forceinline__ float rx_dot(const T* __restrict__ wrow, const float* __restrict__ a, int K, int lane) {
    constexpr int VN = rx_vec<T>::N;
    typedef typename rx_vec<T>::type vec_t;
    float acc = 0.f;
    if (VEC) {
        for (int k = lane * VN; k < K; k += 64 * VN) {
            const vec_t w = *(const vec_t*)(wrow + k);
#pragma unroll
            for (int i = 0; i < VN; ++i) acc = fmaf(to_f32<T>(w[i]), a[k + i], acc);
        }
    } else {
        for (int k = lane; k < K; k += 64) acc = fmaf(to_f32<T>(wrow[k]), a[k], acc);
    }
    return wave_sum(acc);
}

// grid (T * top, ceil(F / 16)), 4 waves, a wave four columns.  LDS: W floats.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void experts_up_kernel(const T* __restrict__ h, const T* __restrict__ w_gu,
                                                         const int* __restrict__ chosen, T* __restrict__ y, int W, int F, int top) {
    extern __shared__ float hs[];
    const int slot = blockIdx.x, t = slot / top;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < W; i += 256) hs[i] = to_f32<T>(h[(size_t)t * W + i]);
    __syncthreads();
    const int e = chosen[slot];
    const T* wg = w_gu + (size_t)e * 2 * F * W;
    const T* wu = wg + (size_t)F * W;
    for (int j = 0; j < 4; ++j) {
        const int f = blockIdx.y * 16 + wave * 4 + j;
        if (f >= F) break;
        const float g = rx_dot<T, VEC>(wg + (size_t)f * W, hs, W, lane);
        const float u = rx_dot<T, VEC>(wu + (size_t)f * W, hs, W, lane);
        if (lane == 0) y[(size_t)slot * F + f] = from_f32<T>(g / (1.0f + expf(-g)) * u);
    }
}

// grid (T, ceil(W / 16)), 4 waves, a wave four columns.  LDS: top * F floats.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void experts_down_kernel(const T* __restrict__ y, const T* __restrict__ w_down,
                                                           const int* __restrict__ chosen, const float* __restrict__ share,
                                                           float* __restrict__ x, int W, int F, int top) {
    extern __shared__ float ys[];
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < top * F; i += 256) ys[i] = to_f32<T>(y[(size_t)t * top * F + i]);
    __syncthreads();
    for (int j = 0; j < 4; ++j) {
        const int n = blockIdx.y * 16 + wave * 4 + j;
        if (n >= W) break;
        float sum = 0.f;
        for (int s = 0; s < top; ++s) {
            const int e = chosen[(size_t)t * top + s];
            const float d = rx_dot<T, VEC>(w_down + ((size_t)e * W + n) * F, ys + (size_t)s * F, F, lane);
            sum = fmaf(share[(size_t)t * top + s], d, sum);
        }
        if (lane == 0) x[(size_t)t * W + n] += sum;
    }
}

extern "C" int br_experts_up(const void* h, const void* w_gu, const int* chosen, void* y, int is_bf16,
                             int T, int W, int F, int top, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (W <= 0 || F <= 0 || top <= 0 || (size_t)W * 4 > 65536 || (F + 15) / 16 > 65535) return BR_BAD_ARG;
    dim3 grid((unsigned)((size_t)T * top), (F + 15) / 16);
    const size_t lds = (size_t)W * sizeof(float);
    const bool vec = W % (is_bf16 ? 8 : 4) == 0;
#define RX_UP(TT, V) experts_up_kernel<TT, V><<<grid, 256, lds, s>>>((const TT*)h, (const TT*)w_gu, chosen, (TT*)y, W, F, top)
    if (is_bf16) { if (vec) RX_UP(bf16, true); else RX_UP(bf16, false); }
    else { if (vec) RX_UP(float, true); else RX_UP(float, false); }
#undef RX_UP
    return br_check_launch();
}

extern "C" int br_experts_down(const void* y, const void* w_down, const int* chosen, const float* share, float* x, int is_bf16,
                               int T, int W, int F, int top, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (W <= 0 || F <= 0 || top <= 0 || (size_t)top * F * 4 > 65536 || (W + 15) / 16 > 65535) return BR_BAD_ARG;
    dim3 grid(T, (W + 15) / 16);
    const size_t lds = (size_t)top * F * sizeof(float);
    const bool vec = F % (is_bf16 ? 8 : 4) == 0;
#define RX_DOWN(TT, V) experts_down_kernel<TT, V><<<grid, 256, lds, s>>>((const TT*)y, (const TT*)w_down, chosen, share, x, W, F, top)
    if (is_bf16) { if (vec) RX_DOWN(bf16, true); else RX_DOWN(bf16, false); }
    else { if (vec) RX_DOWN(float, true); else RX_DOWN(float, false); }
#undef RX_DOWN
    return br_check_launch();
}

// ------------------------------------------------------------ expert by expert -----
// The (token, slot) pairs grouped by expert: first[e] .. first[e + 1] - 1 are the places of expert e's pairs in
// `order` (pair numbers t * top + s), and place[pair] is where a pair went.  One workgroup: counts in LDS, a scan by
// one thread, places handed out by counters.  Which of an expert's pairs comes first is left to the counters; a
// pair's output does not depend on its place.
__global__ __launch_bounds__(1024) void experts_sort_kernel(const int* __restrict__ chosen, int* __restrict__ first,
                                                            int* __restrict__ order, int* __restrict__ place, int n, int E) {
    extern __shared__ int cnt[];                   // [E] counts, then [E] counters
    int* cur = cnt + E;
    for (int e = threadIdx.x; e < E; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += 1024) atomicAdd(&cnt[chosen[i]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0;
        for (int e = 0; e < E; ++e) { first[e] = at; cur[e] = at; at += cnt[e]; }
        first[E] = at;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += 1024) {
        const int p = atomicAdd(&cur[chosen[i]], 1);
        order[p] = i;
        place[i] = p;
    }
}

extern "C" int br_experts_sort(const int* chosen, int* first, int* order, int* place, int n, int E, hipStream_t s) {
    if (n <= 0) return BR_OK;
    if (E <= 0 || E > 4096) return BR_BAD_ARG;
    experts_sort_kernel<<<1, 1024, 2 * E * sizeof(int), s>>>(chosen, first, order, place, n, E);
    return br_check_launch();
}

// rows[p, :] = h[order[p] / top, :]: the tokens' rows in the experts' order.  grid (pairs), 256 threads.
template <typename T>
__global__ __launch_bounds__(256) void experts_gather_kernel(const T* __restrict__ h, const int* __restrict__ order,
                                                             T* __restrict__ rows, int W, int top) {
    const T* src = h + (size_t)(order[blockIdx.x] / top) * W;
    T* dst = rows + (size_t)blockIdx.x * W;
    for (int i = threadIdx.x; i < W; i += 256) dst[i] = src[i];
}

extern "C" int br_experts_gather(const void* h, const int* order, void* rows, int is_bf16, int n, int W, int top, hipStream_t s) {
    if (n <= 0) return BR_OK;
    if (W <= 0 || top <= 0) return BR_BAD_ARG;
    if (is_bf16) experts_gather_kernel<bf16><<<n, 256, 0, s>>>((const bf16*)h, order, (bf16*)rows, W, top);
    else experts_gather_kernel<float><<<n, 256, 0, s>>>((const float*)h, order, (float*)rows, W, top);
    return br_check_launch();
}

// x[t, :] += sum_s share[t, s] * out[place[t * top + s], :] with out the experts' float outputs in their order;
// slots in slot order.  grid (T, ceil(W / 256)).
__global__ __launch_bounds__(256) void experts_combine_kernel(const float* __restrict__ out, const int* __restrict__ place,
                                                              const float* __restrict__ share, float* __restrict__ x, int W, int top) {
    const int t = blockIdx.x, i = blockIdx.y * 256 + threadIdx.x;
    if (i >= W) return;
    float sum = 0.f;
    for (int s = 0; s < top; ++s)
        sum = fmaf(share[(size_t)t * top + s], out[(size_t)place[(size_t)t * top + s] * W + i], sum);
    x[(size_t)t * W + i] += sum;
}

extern "C" int br_experts_combine(const float* out, const int* place, const float* share, float* x, int T, int W, int top,
                                  hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (W <= 0 || top <= 0 || (W + 255) / 256 > 65535) return BR_BAD_ARG;
    experts_combine_kernel<<<dim3(T, (W + 255) / 256), 256, 0, s>>>(out, place, share, x, W, top);
    return br_check_launch();
}

// ------------------------------------------- few tokens, every expert read once -----
// bfloat16 on the matrix cores, for steps whose pairs were grouped by `sort` on the device (nothing comes back to
// the host, so the step can be recorded): a workgroup owns 32 output rows of one expert's matrix and walks that
// expert's pairs 32 at a time, so an expert's weights are read once per 32 of its pairs instead of once per pair.
// Its four waves share k (wave w takes the k-steps of 16 numbered w, w + 4, ...), v_mfma_f32_32x32x16_bf16 with
// the weight rows as the first operand, both operands straight from memory; the waves' sums meet in LDS in wave
// order.  Experts without pairs cost a workgroup a load and a compare.
//
// `up`: rows of h gathered through `order` (pair -> token = pair / top), gate and up rows of the same f in the same
// lane, y[p, f] = silu(g) * u in the experts' order.  grid (E, ceil(F / 32)).
__global__ __launch_bounds__(256) void experts_up_grouped_kernel(const bf16* __restrict__ h, const bf16* __restrict__ w_gu,
                                                                 const int* __restrict__ first, const int* __restrict__ order,
                                                                 bf16* __restrict__ y, int W, int F, int top) {
    __shared__ float red[3][2][16][64];
    const int e = blockIdx.x, f0 = blockIdx.y * 32;
    const int p0 = first[e], p1 = first[e + 1];
    if (p0 >= p1) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 31, g = lane >> 5;
    const int f = f0 + c;
    const bf16* wg = w_gu + ((size_t)e * 2 * F + (f < F ? f : F - 1)) * W;
    const bf16* wu = wg + (size_t)F * W;
    bf16x8 zero;
#pragma unroll
    for (int i = 0; i < 8; ++i) zero[i] = (bf16)0.f;
    for (int pb = p0; pb < p1; pb += 32) {
        const int p = pb + c;
        const bf16* arow = h + (size_t)(order[p < p1 ? p : p1 - 1] / top) * W;
        f32x16 ag, au;
#pragma unroll
        for (int r = 0; r < 16; ++r) { ag[r] = 0.f; au[r] = 0.f; }
        for (int k0 = wave * 16; k0 < W; k0 += 64) {
            const int k = k0 + 8 * g;
            const bool on = k < W;
            const bf16x8 af = (on && p < p1) ? *(const bf16x8*)(arow + k) : zero;
            const bf16x8 gf = (on && f < F) ? *(const bf16x8*)(wg + k) : zero;
            const bf16x8 uf = (on && f < F) ? *(const bf16x8*)(wu + k) : zero;
            ag = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gf, af, ag, 0, 0, 0);
            au = __builtin_amdgcn_mfma_f32_32x32x16_bf16(uf, af, au, 0, 0, 0);
        }
        if (wave > 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) { red[wave - 1][0][r][lane] = ag[r]; red[wave - 1][1][r][lane] = au[r]; }
        }
        __syncthreads();
        if (wave == 0 && p < p1) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float gs = ((ag[r] + red[0][0][r][lane]) + red[1][0][r][lane]) + red[2][0][r][lane];
                const float us = ((au[r] + red[0][1][r][lane]) + red[1][1][r][lane]) + red[2][1][r][lane];
                const int ff = f0 + 8 * (r >> 2) + 4 * g + (r & 3);
                if (ff < F) y[(size_t)p * F + ff] = (bf16)(gs / (1.0f + expf(-gs)) * us);
            }
        }
        __syncthreads();
    }
}

// `down`: out[p, n] = W_d[e] y[p, :] as float for the pairs in the experts' order (`combine` adds them to the rows).
// grid (E, ceil(W / 32)).
__global__ __launch_bounds__(256) void experts_down_grouped_kernel(const bf16* __restrict__ y, const bf16* __restrict__ w_down,
                                                                   const int* __restrict__ first, float* __restrict__ out,
                                                                   int W, int F) {
    __shared__ float red[3][16][64];
    const int e = blockIdx.x, n0 = blockIdx.y * 32;
    const int p0 = first[e], p1 = first[e + 1];
    if (p0 >= p1) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 31, g = lane >> 5;
    const int n = n0 + c;
    const bf16* wr = w_down + ((size_t)e * W + (n < W ? n : W - 1)) * F;
    bf16x8 zero;
#pragma unroll
    for (int i = 0; i < 8; ++i) zero[i] = (bf16)0.f;
    for (int pb = p0; pb < p1; pb += 32) {
        const int p = pb + c;
        const bf16* arow = y + (size_t)(p < p1 ? p : p1 - 1) * F;
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
        for (int k0 = wave * 16; k0 < F; k0 += 64) {
            const int k = k0 + 8 * g;
            const bool on = k < F;
            const bf16x8 af = (on && p < p1) ? *(const bf16x8*)(arow + k) : zero;
            const bf16x8 wf = (on && n < W) ? *(const bf16x8*)(wr + k) : zero;
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, af, acc, 0, 0, 0);
        }
        if (wave > 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) red[wave - 1][r][lane] = acc[r];
        }
        __syncthreads();
        if (wave == 0 && p < p1) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int nn = n0 + 8 * (r >> 2) + 4 * g + (r & 3);
                if (nn < W) out[(size_t)p * W + nn] = ((acc[r] + red[0][r][lane]) + red[1][r][lane]) + red[2][r][lane];
            }
        }
        __syncthreads();
    }
}

// Whether the grouped kernels take these sizes: rows of 16 bytes' multiples.
extern "C" int br_experts_grouped_takes(int W, int F) { return W > 0 && F > 0 && W % 8 == 0 && F % 8 == 0; }

extern "C" int br_experts_up_grouped(const void* h, const void* w_gu, const int* first, const int* order, void* y, int E,
                                     int W, int F, int top, hipStream_t s) {
    if (!br_experts_grouped_takes(W, F) || E <= 0 || top <= 0 || (F + 31) / 32 > 65535) return BR_BAD_ARG;
    experts_up_grouped_kernel<<<dim3(E, (F + 31) / 32), 256, 0, s>>>((const bf16*)h, (const bf16*)w_gu, first, order, (bf16*)y, W, F, top);
    return br_check_launch();
}

extern "C" int br_experts_down_grouped(const void* y, const void* w_down, const int* first, float* out, int E, int W, int F,
                                       hipStream_t s) {
    if (!br_experts_grouped_takes(W, F) || E <= 0 || (W + 31) / 32 > 65535) return BR_BAD_ARG;
    experts_down_grouped_kernel<<<dim3(E, (W + 31) / 32), 256, 0, s>>>((const bf16*)y, (const bf16*)w_down, first, out, W, F);
    return br_check_launch();
}

// ------------------------------------------- many tokens, all experts in one launch -----
// C[p, :] = W[e] A[p, :] for the pairs p of every expert e in the experts' order (A's rows lie in that order).
// bfloat16 on the matrix cores: a workgroup owns 128 pairs of ONE expert x 128 outputs; which expert and which of its
// pairs follows from `first` (the workgroup's number counts the experts' tiles of 128 pairs in turn; numbers beyond
// the last tile leave at once).  K goes 64 at a time through two LDS stages (rows 144 bytes apart so that a lane's
// 16-byte reads spread over the banks), the next stage's rows in registers while the current one is multiplied, one
// barrier a stage; four waves as 2 x 2, each 64 pairs x 64 outputs in four blocks of v_mfma_f32_32x32x16_bf16 with
// the weight rows as the first operand.  grid (ceil(pairs / 128) + E, ceil(N / 128)).  K in steps of 8.
#define RX_KT 64                   // k a stage
#define RX_LD (RX_KT + 8)          // elements from one LDS row to the next
template <typename OutT>
__global__ __launch_bounds__(256, 2) void experts_gemm_kernel(const bf16* __restrict__ A, const bf16* __restrict__ Wt,
                                                              const int* __restrict__ first, OutT* __restrict__ C, int E, int N, int K) {
    constexpr int TPR = RX_KT / 8;             // threads that bring one row of a stage
    constexpr int RPP = 256 / TPR;             // rows a pass of the workgroup brings
    constexpr int NP = 128 / RPP;              // passes a tile
    __shared__ __attribute__((aligned(16))) bf16 As[2][128][RX_LD];
    __shared__ __attribute__((aligned(16))) bf16 Ws[2][128][RX_LD];
    int tile = blockIdx.x, e = 0, p0 = 0, p1 = 0;
    bool found = false;
    for (e = 0; e < E; ++e) {
        const int a = first[e], b = first[e + 1], nt = (b - a + 127) >> 7;
        if (tile < nt) { p0 = a + tile * 128; p1 = b; found = true; break; }
        tile -= nt;
    }
    if (!found) return;
    const int n0 = blockIdx.y * 128;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1, c = lane & 31, g = lane >> 5;
    const int lr = tid / TPR, kc = (tid % TPR) * 8;
    bool va[NP], vw[NP];
    const bf16* ap[NP];
    const bf16* wp[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        va[i] = p0 + lr + i * RPP < p1;
        vw[i] = n0 + lr + i * RPP < N;
        ap[i] = A + (size_t)(va[i] ? p0 + lr + i * RPP : p1 - 1) * K + kc;
        wp[i] = Wt + ((size_t)e * N + (vw[i] ? n0 + lr + i * RPP : N - 1)) * K + kc;
    }
    bf16x8 zero;
#pragma unroll
    for (int i = 0; i < 8; ++i) zero[i] = (bf16)0.f;
    bf16x8 ra[NP], rw[NP];
    auto fetch = [&](int k0) {
        const bool on = k0 + kc < K;
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            ra[i] = (on && va[i]) ? *(const bf16x8*)(ap[i] + k0) : zero;
            rw[i] = (on && vw[i]) ? *(const bf16x8*)(wp[i] + k0) : zero;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            *(bf16x8*)&As[buf][lr + i * RPP][kc] = ra[i];
            *(bf16x8*)&Ws[buf][lr + i * RPP][kc] = rw[i];
        }
    };
    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    fetch(0);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += RX_KT) {
        const bool more = k0 + RX_KT < K;
        if (more) fetch(k0 + RX_KT);
#pragma unroll
        for (int kk = 0; kk < RX_KT / 16; ++kk) {
            bf16x8 af[2], wf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                af[i] = *(const bf16x8*)&As[buf][wm * 64 + i * 32 + c][kk * 16 + 8 * g];
                wf[i] = *(const bf16x8*)&Ws[buf][wn * 64 + i * 32 + c][kk * 16 + 8 * g];
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[i], af[j], acc[i][j], 0, 0, 0);
        }
        if (more) stash(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int p = p0 + wm * 64 + j * 32 + c;
        if (p >= p1) continue;
        OutT* crow = C + (size_t)p * N;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int n = n0 + wn * 64 + i * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
                if (n < N) crow[n] = from_f32<OutT>(acc[i][j][r]);
            }
    }
}

extern "C" int br_experts_gemm(const void* A, const void* Wt, const int* first, void* C, int out_is_bf16, int pairs, int E,
                               int N, int K, hipStream_t s) {
    if (pairs <= 0) return BR_OK;
    if (E <= 0 || N <= 0 || K <= 0 || K % 8 || ((uintptr_t)A % 16) || ((uintptr_t)Wt % 16) || (N + 127) / 128 > 65535) return BR_BAD_ARG;
    dim3 grid((pairs + 127) / 128 + E, (N + 127) / 128);
    if (out_is_bf16) experts_gemm_kernel<bf16><<<grid, 256, 0, s>>>((const bf16*)A, (const bf16*)Wt, first, (bf16*)C, E, N, K);
    else experts_gemm_kernel<float><<<grid, 256, 0, s>>>((const bf16*)A, (const bf16*)Wt, first, (float*)C, E, N, K);
    return br_check_launch();
}
