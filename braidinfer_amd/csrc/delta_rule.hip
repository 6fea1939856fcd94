// Recurrences over an outer-product state with one decay number per head and token, state in float:
// for a head with d key channels and e value channels (S is d x e, starts at zero),
//
//     gated delta rule:   S <- g_t S;  u_t = beta_t (v_t - S^T k_t);  S <- S + k_t u_t^T;  o_t = S^T q_t
//     decayed outer sum:  S <- g S + k_t v_t^T;                                            o_t = S^T q_t
//
// (the read-out sees the current token's write in both).  Column c of S follows
// S[:, c] <- g S[:, c] + k (beta (v[c] - k . S[:, c])) and never meets another column, so the work is cut by
// (sequence, head, 16 columns) and walked like the other recurrences of this library: the state lies in a slot
// as `glr_scan_kernel` keeps it, a lane holds RPL rows of one column in registers, the tokens' rows come TC at a
// time through two LDS stages with the next chunk in flight, and a token costs a lane two sums over its 16 row
// groups (k . S for the correction, q . S for the read-out) by moves between neighbouring lanes in a fixed order.
//
// Beside the scan: `conv_prepare` (a short causal convolution over time per channel with the last inputs kept per
// sequence, silu, unit length per head, the decay and the write strength from their float sums) and
// `conv_keep` (the inputs a sequence's next step needs).
#include "common.h"

#define DR_MAX_EPL 8      // head widths up to 64 * DR_MAX_EPL
#define DR_MAX_TAPS 16

__device__ __forceinline__ float dr_row16_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    return v;
}

__device__ __forceinline__ float dr_silu(float z) { return z / (1.0f + expf(-z)); }

// ------------------------------------------------------------------- prepare -------
// rows [T, width] float, the projections' sums: q (G heads of d) | k (G of d) | v (H of e) | b (H) | a (H) | ...
// One wave per (token, head row) with head rows = G query heads, G key heads, H value heads; four waves a workgroup.  Channel ch of the
// C = 2 G d + H e convolved channels is column ch of `rows`; taps [C, n] float, the last column the current token's;
// `kept` holds per slot the last n - 1 inputs of every channel, [n - 1][C] (zeros in a new slot).
// Out: qo, ko [T, G d] (silu, unit length per head, q times d^-1/2), vo [T, H e] (silu), gb [T, 2 H]:
// g = exp(-exp(A_log) softplus(a + dt_bias)) then beta = sigmoid(b).
__global__ __launch_bounds__(256) void dr_conv_prepare_kernel(
    const float* __restrict__ rows, int width, const float* __restrict__ taps, int n_taps,
    const float* __restrict__ kept, size_t kept_stride, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, float* __restrict__ qo, float* __restrict__ ko, float* __restrict__ vo,
    float* __restrict__ gb, int T, int G, int H, int d, int e) {
    const int n_hr = 2 * G + H;
    const long long unit = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);          // a wave a (token, head row)
    if (unit >= (long long)T * n_hr) return;
    const int t = (int)(unit / n_hr), hr = (int)(unit - (long long)t * n_hr), lane = threadIdx.x & 63;
    const bool is_q = hr < G, is_k = !is_q && hr < 2 * G;
    const int head = is_q ? hr : (is_k ? hr - G : hr - 2 * G);
    const int n = (is_q || is_k) ? d : e;
    const int C = 2 * G * d + H * e;
    const int col0 = is_q ? head * d : (is_k ? G * d + head * d : 2 * G * d + head * e);
    const int b = seq_of_token[t];
    const int slot = slots[b], t0 = cu_seqlens[b];
    const int i_in_step = t - t0;
    float v[DR_MAX_EPL];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < DR_MAX_EPL; ++j) {
        const int i = lane + 64 * j;
        v[j] = 0.f;
        if (i < n) {
            const int ch = col0 + i;
            float acc = 0.f;
            for (int x = 0; x < n_taps; ++x) {
                const int ii = i_in_step - (n_taps - 1) + x;          // the input's place in the step
                float in;
                if (ii >= 0) in = rows[(size_t)(t0 + ii) * width + ch];
                else in = slot >= 0 ? kept[(size_t)slot * kept_stride + (size_t)(n_taps - 1 + ii) * C + ch] : 0.f;
                acc = fmaf(taps[(size_t)ch * n_taps + x], in, acc);
            }
            v[j] = dr_silu(acc);
            ss = fmaf(v[j], v[j], ss);
        }
    }
    float mult = 1.f;
    if (is_q || is_k) {
        mult = 1.0f / sqrtf(wave_sum(ss) + 1e-6f);
        if (is_q) mult *= 1.0f / sqrtf((float)d);
    }
    float* dst = is_q ? qo + (size_t)t * G * d + head * d : (is_k ? ko + (size_t)t * G * d + head * d
                                                                   : vo + (size_t)t * H * e + head * e);
#pragma unroll
    for (int j = 0; j < DR_MAX_EPL; ++j) {
        const int i = lane + 64 * j;
        if (i < n) dst[i] = v[j] * mult;
    }
    if (!is_q && !is_k && lane == 0) {
        const float braw = rows[(size_t)t * width + C + head];
        const float araw = rows[(size_t)t * width + C + H + head] + dt_bias[head];
        const float sp = araw > 20.f ? araw : log1pf(expf(araw));
        gb[(size_t)t * 2 * H + head] = expf(-expf(a_log[head]) * sp);
        gb[(size_t)t * 2 * H + H + head] = 1.0f / (1.0f + expf(-braw));
    }
}

// The same with four channels a lane through 16-byte loads, for widths that are multiples of 4 (d, e, `width`, the kept
// rows' stride; 16-byte aligned pointers): `taps_t` [n, C] holds the taps with the channels side by side.  LPH lanes a
// (token, head row), 64 / LPH of them a wave: 16 lanes for heads of up to 64 channels, 32 up to 128, else 64.
template <int LPH>
__global__ __launch_bounds__(256) void dr_conv_prepare_vec_kernel(
    const float* __restrict__ rows, int width, const float* __restrict__ taps_t, int n_taps,
    const float* __restrict__ kept, size_t kept_stride, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, float* __restrict__ qo, float* __restrict__ ko, float* __restrict__ vo,
    float* __restrict__ gb, int T, int G, int H, int d, int e) {
    constexpr int NJ = LPH == 64 ? DR_MAX_EPL / 4 : 1;
    const int n_hr = 2 * G + H;
    const int lane = threadIdx.x & 63, l = lane % LPH;
    const long long unit = ((long long)blockIdx.x * 4 + (threadIdx.x >> 6)) * (64 / LPH) + lane / LPH;
    const bool on = unit < (long long)T * n_hr;          // lanes behind the last row go along for the sums and write nothing
    const int t = on ? (int)(unit / n_hr) : 0, hr = on ? (int)(unit - (long long)t * n_hr) : 0;
    const bool is_q = hr < G, is_k = !is_q && hr < 2 * G;
    const int head = is_q ? hr : (is_k ? hr - G : hr - 2 * G);
    const int n = (is_q || is_k) ? d : e;
    const int C = 2 * G * d + H * e;
    const int col0 = is_q ? head * d : (is_k ? G * d + head * d : 2 * G * d + head * e);
    const int b = seq_of_token[t];
    const int slot = slots[b], t0 = cu_seqlens[b];
    const int i_in_step = t - t0;
    f32x4 v[NJ];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int i = 4 * l + 4 * LPH * j;
        v[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (on && i < n) {
            const int ch = col0 + i;
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            for (int x = 0; x < n_taps; ++x) {
                const int ii = i_in_step - (n_taps - 1) + x;          // the input's place in the step
                f32x4 in = {0.f, 0.f, 0.f, 0.f};
                if (ii >= 0) in = *(const f32x4*)(rows + (size_t)(t0 + ii) * width + ch);
                else if (slot >= 0) in = *(const f32x4*)(kept + (size_t)slot * kept_stride + (size_t)(n_taps - 1 + ii) * C + ch);
                const f32x4 w = *(const f32x4*)(taps_t + (size_t)x * C + ch);
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[c] = fmaf(w[c], in[c], acc[c]);
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                v[j][c] = dr_silu(acc[c]);
                ss = fmaf(v[j][c], v[j][c], ss);
            }
        }
    }
#pragma unroll
    for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, WAVE);          // over the row's lanes, in a fixed order
    if (!on) return;
    float mult = 1.f;
    if (is_q || is_k) {
        mult = 1.0f / sqrtf(ss + 1e-6f);
        if (is_q) mult *= 1.0f / sqrtf((float)d);
    }
    float* dst = is_q ? qo + (size_t)t * G * d + head * d : (is_k ? ko + (size_t)t * G * d + head * d
                                                                   : vo + (size_t)t * H * e + head * e);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int i = 4 * l + 4 * LPH * j;
        if (i < n) {
            f32x4 out;
#pragma unroll
            for (int c = 0; c < 4; ++c) out[c] = v[j][c] * mult;
            *(f32x4*)(dst + i) = out;
        }
    }
    if (!is_q && !is_k && l == 0) {
        const float braw = rows[(size_t)t * width + C + head];
        const float araw = rows[(size_t)t * width + C + H + head] + dt_bias[head];
        const float sp = araw > 20.f ? araw : log1pf(expf(araw));
        gb[(size_t)t * 2 * H + head] = expf(-expf(a_log[head]) * sp);
        gb[(size_t)t * 2 * H + H + head] = 1.0f / (1.0f + expf(-braw));
    }
}

// After the step: every sequence's last n - 1 inputs into its slot.  grid (B, ceil(C / 256)).
__global__ __launch_bounds__(256) void dr_conv_keep_kernel(const float* __restrict__ rows, int width, int n_taps,
                                                           float* __restrict__ kept, size_t kept_stride,
                                                           const int* __restrict__ cu_seqlens,
                                                           const int* __restrict__ slots, int C) {
    const int b = blockIdx.x, ch = blockIdx.y * 256 + threadIdx.x;
    const int slot = slots[b];
    if (ch >= C || slot < 0) return;
    const int t0 = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t0, keep = n_taps - 1;
    float* st = kept + (size_t)slot * kept_stride + ch;
    float old[DR_MAX_TAPS];
    for (int j = 0; j < keep; ++j) old[j] = st[(size_t)j * C];
    for (int j = 0; j < keep; ++j) {
        const int ii = n_new - keep + j;
        st[(size_t)j * C] = ii >= 0 ? rows[(size_t)(t0 + ii) * width + ch] : old[keep + ii];
    }
}

extern "C" int br_dr_conv_prepare(const float* rows, int width, const float* taps, const float* taps_t, int n_taps, float* kept,
                                  size_t kept_stride, const float* a_log, const float* dt_bias, const int* seq_of_token,
                                  const int* cu_seqlens, const int* slots, float* qo, float* ko, float* vo, float* gb,
                                  int T, int B, int G, int H, int d, int e, hipStream_t s) {
    if (T <= 0 || B <= 0) return BR_OK;
    const long long C = 2LL * G * d + (long long)H * e;
    if (G <= 0 || H <= 0 || H % G || d <= 0 || e <= 0 || d > 64 * DR_MAX_EPL || e > 64 * DR_MAX_EPL || n_taps < 1 ||
        n_taps > DR_MAX_TAPS || width < C + 2 * H || ((long long)T * (2 * G + H) + 3) / 4 > 0x7fffffffLL || B > 65535 ||
        (C + 255) / 256 > 65535 ||
        (n_taps > 1 && (!kept || kept_stride < (size_t)(n_taps - 1) * C)) || !a_log || !dt_bias)
        return BR_BAD_ARG;
    const unsigned blocks = (unsigned)(((long long)T * (2 * G + H) + 3) / 4);
    auto at16 = [](const void* p) { return ((uintptr_t)p % 16) == 0; };
    const bool vec = taps_t && d % 4 == 0 && e % 4 == 0 && width % 4 == 0 && at16(rows) && at16(taps_t) && at16(qo) && at16(ko) &&
                     at16(vo) && (n_taps == 1 || (kept_stride % 4 == 0 && at16(kept)));
    if (vec) {
        const int widest = d > e ? d : e, lph = widest <= 64 ? 16 : (widest <= 128 ? 32 : 64);
        const unsigned vblocks = (unsigned)(((long long)T * (2 * G + H) + 4 * (64 / lph) - 1) / (4 * (64 / lph)));
#define DR_PREP(L) dr_conv_prepare_vec_kernel<L><<<vblocks, 256, 0, s>>>(rows, width, taps_t, n_taps, kept, kept_stride, a_log, dt_bias, \
                                                                        seq_of_token, cu_seqlens, slots, qo, ko, vo, gb, T, G, H, d, e)
        if (lph == 16) DR_PREP(16); else if (lph == 32) DR_PREP(32); else DR_PREP(64);
#undef DR_PREP
    }
    else dr_conv_prepare_kernel<<<blocks, 256, 0, s>>>(rows, width, taps, n_taps, kept, kept_stride, a_log, dt_bias, seq_of_token,
                                                 cu_seqlens, slots, qo, ko, vo, gb, T, G, H, d, e);
    int rc = br_check_launch();
    if (rc != BR_OK || n_taps == 1) return rc;
    dr_conv_keep_kernel<<<dim3(B, (unsigned)((C + 255) / 256)), 256, 0, s>>>(rows, width, n_taps, kept, kept_stride, cu_seqlens,
                                                                           slots, (int)C);
    return br_check_launch();
}

// x[t, :n] <- silu(x[t, :n]) in place on float rows `stride` apart (projections' sums that go on as activations: done
// once here, not by every workgroup of a scan that reads them).  VEC: four a thread, for n, stride and pointer in fours.
template <bool VEC>
__global__ __launch_bounds__(256) void dr_silu_rows_kernel(float* __restrict__ x, size_t stride, int n, size_t total) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    if (VEC) {
        const size_t per = (size_t)n / 4, t = i / per, c = (i - t * per) * 4;
        f32x4* p = (f32x4*)(x + t * stride + c);
        f32x4 v = *p;
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = dr_silu(v[k]);
        *p = v;
    } else {
        const size_t t = i / n, c = i - t * n;
        float* p = x + t * stride + c;
        *p = dr_silu(*p);
    }
}

extern "C" int br_silu_rows(float* x, size_t stride, int T, int n, hipStream_t s) {
    if (T <= 0 || n <= 0) return BR_OK;
    if (stride < (size_t)n) return BR_BAD_ARG;
    const bool vec = n % 4 == 0 && stride % 4 == 0 && ((uintptr_t)x % 16) == 0;
    const size_t total = vec ? (size_t)T * (n / 4) : (size_t)T * n;
    const size_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffULL) return BR_BAD_ARG;
    if (vec) dr_silu_rows_kernel<true><<<(unsigned)blocks, 256, 0, s>>>(x, stride, n, total);
    else dr_silu_rows_kernel<false><<<(unsigned)blocks, 256, 0, s>>>(x, stride, n, total);
    return br_check_launch();
}

// q and k rows (float sums of their projections, rows `stride` apart, `heads` heads of d channels each) turned in place
// by their tokens' positions: of the first `rd` channels of a head, channel i < rd / 2 and channel i + rd / 2 form
// a pair that is turned by the angle whose cosine and sine are cs[t, i], sn[t, i] ((u, v) -> (u c - v s, v c + u s));
// the other channels pass.  Every channel of q is then multiplied by `q_mul` and every channel of k by `k_mul`.
// A thread a channel below rd / 2 (it owns the pair) or from rd on; grid over T * heads * (d - rd / 2) threads.
__global__ __launch_bounds__(256) void dr_rotate_rows_kernel(float* __restrict__ q, float* __restrict__ k, size_t stride,
                                                             const float* __restrict__ cs, const float* __restrict__ sn,
                                                             int rd, int heads, int d, float q_mul, float k_mul, size_t total) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int half = rd >> 1, per = d - half;
    const size_t th = i / per;
    const int j = (int)(i - th * per);
    const size_t t = th / heads;
    const int h = (int)(th - t * heads);
    float* qr = q + t * stride + (size_t)h * d;
    float* kr = k + t * stride + (size_t)h * d;
    if (j < half) {
        const float c = cs[t * half + j], s_ = sn[t * half + j];
        const float qu = qr[j], qv = qr[j + half], ku = kr[j], kv = kr[j + half];
        qr[j] = (qu * c - qv * s_) * q_mul;
        qr[j + half] = (qv * c + qu * s_) * q_mul;
        kr[j] = (ku * c - kv * s_) * k_mul;
        kr[j + half] = (kv * c + ku * s_) * k_mul;
    } else {
        const int ch = j + half;                    // channels from rd on
        qr[ch] *= q_mul;
        kr[ch] *= k_mul;
    }
}

extern "C" int br_dr_rotate_rows(float* q, float* k, size_t stride, const float* cs, const float* sn, int rd, int T, int heads,
                                 int d, float q_mul, float k_mul, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (heads <= 0 || d <= 0 || rd < 0 || (rd & 1) || rd > d || stride < (size_t)heads * d || (rd > 0 && (!cs || !sn))) return BR_BAD_ARG;
    const size_t total = (size_t)T * heads * (d - rd / 2);
    const size_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffULL) return BR_BAD_ARG;
    dr_rotate_rows_kernel<<<(unsigned)blocks, 256, 0, s>>>(q, k, stride, cs, sn, rd, heads, d, q_mul, k_mul, total);
    return br_check_launch();
}

// ---------------------------------------------------------------------- scan -------
// q, k: float rows `qk_stride` apart, head kh's d channels at kh * d (kh = h / (H / G): G heads of keys serve H
// heads of values); v: rows `v_stride` apart, head h's e channels at h * e.  DELTA: g and beta per token and
// head from `gb` (rows `gb_stride` apart, g at [h], beta at [H + h]); else the head's one decay `g_head[h]` and
// u = v.  SILU: q, k and v are the projections' float sums and pass silu on their way into LDS.
// grid (sequences, heads, ceil(e / 16)), 256 threads; a slot's state as `glr_state_shape` says.
// LOCAL (the first pass over a long prompt cut into pieces, see `br_dr_scan_pieces`): the state starts at zero, nothing
// is written to o, and the last state goes to the piece's scratch.
template <int RPL, int TC, bool DELTA, bool SILU, bool LOCAL>
__global__ __launch_bounds__(256) void dr_scan_kernel(
    const float* __restrict__ q, const float* __restrict__ k, size_t qk_stride, const float* __restrict__ v,
    size_t v_stride, const float* __restrict__ gb, size_t gb_stride, const float* __restrict__ g_head,
    float* __restrict__ o, float* __restrict__ state, size_t slot_stride, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, int H, int G, int d, int e) {
    constexpr int DP = RPL * 16;
    constexpr int NL = TC * DP / 1024;
    extern __shared__ float lds[];
    float* kL = lds;                               // [2][TC][DP]
    float* qL = kL + 2 * TC * DP;                  // [2][TC][DP]
    float* vL = qL + 2 * TC * DP;                  // [2][TC][16]
    float* gL = vL + 2 * TC * 16;                  // [2][TC][2]
    const int s = blockIdx.x, h = blockIdx.y, cb16 = blockIdx.z;
    const int kh = h / (H / G);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cg = lane >> 4, g = lane & 15;
    const int cb4 = cb16 * 4 + wave, c = cb4 * 4 + cg;
    const int slot = slots[s];
    const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
    const bool live = c < e;
    const int he = H * e;
    if (slot < 0) {                                // padding: no state behind it; its rows of o are zero
        if (!LOCAL && g == 0 && live) for (int t = t0; t < t1; ++t) o[(size_t)t * he + h * e + c] = 0.f;
        return;
    }
    const int ncb4 = (e + 3) >> 2;
    float* S = state + (size_t)slot * slot_stride + (((size_t)h * ncb4 + cb4) * RPL) * 64 + lane;
    float st[RPL];
#pragma unroll
    for (int r = 0; r < RPL; ++r) st[r] = (!LOCAL && cb4 < ncb4) ? S[(size_t)r * 64] : 0.f;
    const float g_fixed = DELTA ? 1.f : g_head[h];
    int l_tt[NL], l_r4[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int idx = tid + 256 * i;
        l_tt[i] = idx / (DP / 4);
        l_r4[i] = (idx % (DP / 4)) * 4;
    }
    const int v_tt = tid >> 4, v_c = cb16 * 16 + (tid & 15);
    float rq[NL][4], rk[NL][4], rv = 0.f, rg = 1.f;

    auto fetch = [&](int tc0) {
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const int t = tc0 + l_tt[i];
            const float* qp = q + (size_t)t * qk_stride + kh * d + l_r4[i];
            const float* kp = k + (size_t)t * qk_stride + kh * d + l_r4[i];
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const bool ok = t < t1 && l_r4[i] + x < d;
                rq[i][x] = ok ? qp[x] : 0.f;
                rk[i][x] = ok ? kp[x] : 0.f;
            }
        }
        const int t = tc0 + v_tt;
        rv = (v_tt < TC && t < t1 && v_c < e) ? v[(size_t)t * v_stride + h * e + v_c] : 0.f;
        if (DELTA) {
            // threads 0 .. 2 TC - 1 bring the chunk's decays and write strengths
            const int gt = tc0 + (tid >> 1);
            rg = (tid < 2 * TC && gt < t1) ? gb[(size_t)gt * gb_stride + (tid & 1) * H + h] : 1.f;
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            f32x4 ko, qo;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const bool real = l_r4[i] + x < d;       // rows behind d: key 0, query 0, so their state stays 0
                ko[x] = real ? (SILU ? dr_silu(rk[i][x]) : rk[i][x]) : 0.f;
                qo[x] = real ? (SILU ? dr_silu(rq[i][x]) : rq[i][x]) : 0.f;
            }
            const size_t at = ((size_t)buf * TC + l_tt[i]) * DP + l_r4[i];
            *(f32x4*)(kL + at) = ko;
            *(f32x4*)(qL + at) = qo;
        }
        if (v_tt < TC) vL[(buf * TC + v_tt) * 16 + (tid & 15)] = SILU ? dr_silu(rv) : rv;
        if (DELTA && tid < 2 * TC) gL[buf * TC * 2 + tid] = rg;
    };

    fetch(t0);
    stage(0);
    __syncthreads();
    int buf = 0;
    float* orow = o + (size_t)t0 * he + h * e + c;
    for (int tc0 = t0; tc0 < t1; tc0 += TC) {
        const bool more = tc0 + TC < t1;
        if (more) fetch(tc0 + TC);
        const int nt = t1 - tc0 < TC ? t1 - tc0 : TC;
        const float* kp = kL + (size_t)buf * TC * DP + g * RPL;
        const float* qp = qL + (size_t)buf * TC * DP + g * RPL;
        const float* vp = vL + buf * TC * 16 + wave * 4 + cg;
        const float* gp = gL + buf * TC * 2;
#pragma unroll 2
        for (int tt = 0; tt < nt; ++tt) {
            const float vc = vp[tt * 16];
            float kr[RPL];
#pragma unroll
            for (int k4 = 0; k4 < RPL / 4; ++k4) {
                const f32x4 kv4 = *(const f32x4*)(kp + (size_t)tt * DP + 4 * k4);
#pragma unroll
                for (int x = 0; x < 4; ++x) kr[4 * k4 + x] = kv4[x];
            }
            float u = vc;
            const float gt = DELTA ? gp[2 * tt] : g_fixed;
            if (DELTA) {
                float part = 0.f;
#pragma unroll
                for (int r = 0; r < RPL; ++r) {
                    st[r] *= gt;
                    part = fmaf(st[r], kr[r], part);
                }
                u = gp[2 * tt + 1] * (vc - dr_row16_sum(part));
            }
            float sum = 0.f;
#pragma unroll
            for (int k4 = 0; k4 < RPL / 4; ++k4) {
                const f32x4 qv4 = *(const f32x4*)(qp + (size_t)tt * DP + 4 * k4);
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const int r = 4 * k4 + x;
                    st[r] = DELTA ? fmaf(kr[r], u, st[r]) : fmaf(gt, st[r], kr[r] * u);
                    sum = fmaf(st[r], qv4[x], sum);
                }
            }
            sum = dr_row16_sum(sum);
            if (!LOCAL && g == 0 && live) orow[0] = sum;
            orow += he;
        }
        if (more) stage(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
    if (cb4 < ncb4) {
#pragma unroll
        for (int r = 0; r < RPL; ++r) S[(size_t)r * 64] = st[r];
    }
}

static inline int dr_rpl(int d) {
    const int r = (d + 15) / 16;
    return r <= 4 ? 4 : (r <= 8 ? 8 : (r <= 16 ? 16 : 32));
}

template <bool LOCAL>
static int dr_scan_launch(const float* q, const float* k, size_t qk_stride, const float* v, size_t v_stride, const float* gb,
                          size_t gb_stride, const float* g_head, float* o, float* state, size_t slot_stride,
                          const int* cu_seqlens, const int* slots, int B, int H, int G, int d, int e, int delta, int silu,
                          hipStream_t s) {
    const int ncb4 = (e + 3) / 4, rpl = dr_rpl(d);
    if (H <= 0 || H > 65535 || G <= 0 || H % G || d <= 0 || e <= 0 || d > 512 || (e + 15) / 16 > 65535 || B > 0x7fffffff ||
        qk_stride < (size_t)G * d || v_stride < (size_t)H * e || slot_stride < (size_t)H * ncb4 * rpl * 64 ||
        (delta && (!gb || gb_stride < (size_t)2 * H)) || (!delta && !g_head) || (LOCAL && delta))
        return BR_BAD_ARG;
    dim3 grid(B, H, (e + 15) / 16);
#define DR_GO(R, TC, D, A) do { \
        const size_t lds = (size_t)(4 * TC * R * 16 + 2 * TC * 16 + 2 * TC * 2) * sizeof(float); \
        dr_scan_kernel<R, TC, D, A, LOCAL><<<grid, 256, lds, s>>>(q, k, qk_stride, v, v_stride, gb, gb_stride, g_head, o, state, slot_stride, \
                                                                 cu_seqlens, slots, H, G, d, e); \
    } while (0)
#define DR_SCAN(R, TC) do { \
        if (delta) { if (LOCAL) return BR_BAD_ARG; if (silu) DR_GO(R, TC, true, true); else DR_GO(R, TC, true, false); } \
        else { if (silu) DR_GO(R, TC, false, true); else DR_GO(R, TC, false, false); } \
    } while (0)
    if (rpl == 4) DR_SCAN(4, 16);
    else if (rpl == 8) DR_SCAN(8, 16);
    else if (rpl == 16) DR_SCAN(16, 8);
    else DR_SCAN(32, 4);
#undef DR_SCAN
#undef DR_GO
    return br_check_launch();
}

// `delta` 1: the gated delta rule with `gb`; 0: the decayed outer sum with `g_head`.  `silu` 1: q, k, v pass silu.
extern "C" int br_dr_scan(const float* q, const float* k, size_t qk_stride, const float* v, size_t v_stride, const float* gb,
                          size_t gb_stride, const float* g_head, float* o, float* state, size_t slot_stride,
                          const int* cu_seqlens, const int* slots, int B, int H, int G, int d, int e, int delta, int silu,
                          hipStream_t s) {
    if (B <= 0) return BR_OK;
    return dr_scan_launch<false>(q, k, qk_stride, v, v_stride, gb, gb_stride, g_head, o, state, slot_stride, cu_seqlens, slots,
                                 B, H, G, d, e, delta, silu, s);
}

// Between the two passes over a prompt cut into `pieces` pieces per sequence, for the decayed outer sum: from the
// sequence's own state s_0 and every piece's local last state L_c, the state each piece starts from,
// s_(c+1) = decay_h^(tokens of piece c) s_c + L_c, written over L_c; the last one becomes the sequence's state.
// grid (sequences, heads * column blocks of 4), block 64.
__global__ __launch_bounds__(64) void dr_carry_kernel(float* __restrict__ state, size_t slot_stride, const int* __restrict__ slots,
                                                      float* __restrict__ piece_state, size_t piece_stride,
                                                      const int* __restrict__ piece_cu, const float* __restrict__ g_head,
                                                      int pieces, int ncb4, int rpl) {
    const int b = blockIdx.x, hc = blockIdx.y, lane = threadIdx.x;
    const int slot = slots[b];
    if (slot < 0) return;
    const float decay = g_head[hc / ncb4];
    for (int k = 0; k < rpl; ++k) {
        const size_t idx = ((size_t)hc * rpl + k) * 64 + lane;
        float sv = state[(size_t)slot * slot_stride + idx];
        for (int c = 0; c < pieces; ++c) {
            const size_t v = (size_t)b * pieces + c;
            const float local = piece_state[v * piece_stride + idx];
            piece_state[v * piece_stride + idx] = sv;
            sv = fmaf(powf(decay, (float)(piece_cu[v + 1] - piece_cu[v])), sv, local);
        }
        state[(size_t)slot * slot_stride + idx] = sv;
    }
}

// The decayed outer sum over a step of long prompts with every sequence cut into `pieces` pieces that run side by side:
// the recurrence is linear in the state, so a piece can be walked from a zero state first (its last state L), the
// pieces' true first states follow from s_(c+1) = decay^n_c s_c + L_c, and a second walk from those writes o.  Twice
// the arithmetic for `pieces` times the workgroups; results differ from the plain walk by the rounding of that one
// combination per piece.  `piece_cu` [B * pieces + 1] cuts the packed tokens (pieces of a sequence in order, empty
// ones allowed), `piece_slots` [B * pieces] is the piece's own number (or -1 for a padding sequence's),
// `piece_state` [B * pieces][state of a slot] is scratch.
extern "C" int br_dr_scan_pieces(const float* q, const float* k, size_t qk_stride, const float* v, size_t v_stride,
                                 const float* g_head, float* o, float* state, size_t slot_stride, const int* slots,
                                 const int* piece_cu, const int* piece_slots, float* piece_state, int B, int pieces, int H,
                                 int d, int e, int silu, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (pieces <= 0 || (long long)B * pieces > 65535 || B > 65535) return BR_BAD_ARG;
    const int ncb4 = (e + 3) / 4, rpl = dr_rpl(d);
    const size_t piece_stride = (size_t)H * ncb4 * rpl * 64;
    int rc = dr_scan_launch<true>(q, k, qk_stride, v, v_stride, nullptr, 0, g_head, o, piece_state, piece_stride, piece_cu,
                                  piece_slots, B * pieces, H, H, d, e, 0, silu, s);
    if (rc != BR_OK) return rc;
    if ((long long)H * ncb4 > 65535 || slot_stride < piece_stride) return BR_BAD_ARG;
    dr_carry_kernel<<<dim3(B, H * ncb4), 64, 0, s>>>(state, slot_stride, slots, piece_state, piece_stride, piece_cu, g_head, pieces,
                                                     ncb4, rpl);
    rc = br_check_launch();
    if (rc != BR_OK) return rc;
    return dr_scan_launch<false>(q, k, qk_stride, v, v_stride, nullptr, 0, g_head, o, piece_state, piece_stride, piece_cu,
                                 piece_slots, B * pieces, H, H, d, e, 0, silu, s);
}
