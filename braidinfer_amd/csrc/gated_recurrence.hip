// A gated linear recurrence per head, state in float: for a head with d query channels and e
// value channels,
//     S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T      (S is d x e, starts at zero)
//     o_t = S_t^T q_t
// with the forget gate f_t in (lower, 1) per channel deciding what stays and what is written
// (no key, no further scale).  The columns of S never meet: column c follows
// S[:, c] <- f * S[:, c] + (1 - f) * v[c], so the work is cut by (sequence, head, 16 columns).
//
// Two kernels: `scan` turns the projections' float sums into q = silu(.) and
// f = lower + (1 - lower) * sigmoid(. + bias) on their way into LDS and walks a sequence's new
// tokens in order from the state its slot holds, leaving the state behind; `head_norm` is the RMS
// norm of every head's output over its e channels.
#include "common.h"

// ----------------------------------------------------------------------- scan ------
// rows [T, 2 * hd + he] are the projections' float sums q | f | v (hd = heads * d).
// grid (sequences, heads, ceil(e / 16)), 256 threads.  A workgroup walks its sequence's new tokens for 16
// columns of one head's state, TC tokens at a time through two LDS stages: while the waves work on one
// chunk, the next chunk's rows are on their way from memory into registers (coalesced, 16 bytes a thread
// where rows are aligned so), and go into the other stage with the gates applied (q = silu(.),
// f = lower + (1 - lower) * sigmoid(. + bias)) behind the chunk's one barrier.  Each wave owns 4 of the 16
// columns and needs no other barrier: lane (cg, g) holds the rows g RPL .. g RPL + RPL - 1 of column cg in
// registers; a token costs it RPL / 4 reads of 16 bytes each of gates and queries from LDS (the same for
// the four columns), one value, 3 RPL multiply-adds and four moves between neighbouring lanes that add the
// 16 row groups' shares of o_t[c] in a fixed order.  Rows from d to 16 RPL are padding: gate 1, query 0, state 0.
//
// A slot's state lies as the lanes hold it: [head][column block of 4][k][lane], S[r][c] at block c / 4,
// k = r % RPL, lane = 16 (c % 4) + r / RPL, so a wave reads and writes 256 contiguous bytes for each k.
// The sum of v over each row of 16 lanes, in every lane of the row, by four data-parallel-primitive moves
// (neighbour, other pair, other quad mirrored, other half mirrored) in a fixed order.
__device__ __forceinline__ float glr_row16_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    return v;
}

//
// LOCAL (the first pass over a long prompt cut into pieces, see `br_glr_scan_pieces`): the state starts at
// zero, nothing is written to o, and beside the piece's last state the products of its gates go to `decay`
// ([sequences of the launch][head][16 RPL], in row order).
template <int RPL, int TC, bool V4, bool LOCAL>
__global__ __launch_bounds__(256) void glr_scan_kernel(
    const float* __restrict__ rows, const float* __restrict__ f_bias, const float* __restrict__ lower,
    float* __restrict__ o, float* __restrict__ state, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, int H, int d, int e, int width, size_t slot_stride, float* __restrict__ decay) {
    constexpr int DP = RPL * 16;                   // rows of a column with padding
    constexpr int NL = TC * DP / 1024;             // groups of 4 rows a thread brings per chunk and array
    extern __shared__ float lds[];
    float* fL = lds;                               // [2][TC][DP]
    float* qL = fL + 2 * TC * DP;                  // [2][TC][DP]
    float* vL = qL + 2 * TC * DP;                  // [2][TC][16]
    const int s = blockIdx.x, h = blockIdx.y, cb16 = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cg = lane >> 4, g = lane & 15;
    const int cb4 = cb16 * 4 + wave, c = cb4 * 4 + cg;
    const int slot = slots[s];
    if (slot < 0) return;
    const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
    const bool live = c < e;
    const int ncb4 = (e + 3) >> 2;
    float* S = state + (size_t)slot * slot_stride + (((size_t)h * ncb4 + cb4) * RPL) * 64 + lane;
    float st[RPL];
#pragma unroll
    for (int k = 0; k < RPL; ++k) st[k] = (!LOCAL && cb4 < ncb4) ? S[(size_t)k * 64] : 0.f;
    float dec[LOCAL ? RPL : 1];
#pragma unroll
    for (int k = 0; k < (LOCAL ? RPL : 1); ++k) dec[k] = 1.f;
    const int hd = H * d;
    // what this thread brings per chunk: group i is rows r4 .. r4 + 3 of token tt
    int l_tt[NL], l_r4[NL];
    float lo4[NL][4], b4[NL][4];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int idx = tid + 256 * i;
        l_tt[i] = idx / (DP / 4);
        l_r4[i] = (idx % (DP / 4)) * 4;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            const int r = l_r4[i] + x;
            lo4[i][x] = (r < d && lower) ? lower[h * d + r] : 0.f;
            b4[i][x] = (r < d && f_bias) ? f_bias[h * d + r] : 0.f;
        }
    }
    const int v_tt = tid >> 4, v_c = cb16 * 16 + (tid & 15);
    float rq[NL][4], rf[NL][4], rv = 0.f;

    auto fetch = [&](int tc0) {                    // rows of the chunk that starts at token tc0, raw, into registers
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const int t = tc0 + l_tt[i];
            const float* qp = rows + (size_t)t * width + h * d + l_r4[i];
            if (V4) {
                f32x4 a = {0.f, 0.f, 0.f, 0.f}, bq = {0.f, 0.f, 0.f, 0.f};
                if (t < t1 && l_r4[i] < d) { a = *(const f32x4*)qp; bq = *(const f32x4*)(qp + hd); }
#pragma unroll
                for (int x = 0; x < 4; ++x) { rq[i][x] = a[x]; rf[i][x] = bq[x]; }
            } else {
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const bool ok = t < t1 && l_r4[i] + x < d;
                    rq[i][x] = ok ? qp[x] : 0.f;
                    rf[i][x] = ok ? qp[hd + x] : 0.f;
                }
            }
        }
        const int t = tc0 + v_tt;
        rv = (v_tt < TC && t < t1 && v_c < e) ? rows[(size_t)t * width + 2 * hd + h * e + v_c] : 0.f;
    };
    auto stage = [&](int buf) {                    // the fetched rows into LDS stage `buf`, gates applied
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            f32x4 qo, fo;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const bool real = l_r4[i] + x < d;
                // exp and reciprocal by the hardware's own instructions (about an ulp each)
                const float z = rq[i][x];
                qo[x] = real ? z * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * z)) : 0.f;
                const float gt = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * (rf[i][x] + b4[i][x])));
                fo[x] = real ? lo4[i][x] + (1.0f - lo4[i][x]) * gt : 1.f;
            }
            *(f32x4*)(qL + ((size_t)buf * TC + l_tt[i]) * DP + l_r4[i]) = qo;
            *(f32x4*)(fL + ((size_t)buf * TC + l_tt[i]) * DP + l_r4[i]) = fo;
        }
        if (v_tt < TC) vL[(buf * TC + v_tt) * 16 + (tid & 15)] = rv;
    };

    fetch(t0);
    stage(0);
    __syncthreads();
    int buf = 0;
    float* orow = o + (size_t)t0 * H * e + h * e + c;
    for (int tc0 = t0; tc0 < t1; tc0 += TC) {
        const bool more = tc0 + TC < t1;
        if (more) fetch(tc0 + TC);
        const int nt = t1 - tc0 < TC ? t1 - tc0 : TC;
        const float* fp = fL + (size_t)buf * TC * DP + g * RPL;
        const float* qp = qL + (size_t)buf * TC * DP + g * RPL;
        const float* vp = vL + buf * TC * 16 + wave * 4 + cg;
#pragma unroll 4
        for (int tt = 0; tt < nt; ++tt) {
            const float vc = vp[tt * 16];
            float sum = 0.f;
#pragma unroll
            for (int k4 = 0; k4 < RPL / 4; ++k4) {
                const f32x4 f = *(const f32x4*)(fp + (size_t)tt * DP + 4 * k4);
                f32x4 qv = {0.f, 0.f, 0.f, 0.f};
                if (!LOCAL) qv = *(const f32x4*)(qp + (size_t)tt * DP + 4 * k4);
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    // f s + (1 - f) v as v + f (s - v): a subtraction and a multiply-add a row
                    st[4 * k4 + x] = fmaf(f[x], st[4 * k4 + x] - vc, vc);
                    if (LOCAL) dec[LOCAL ? 4 * k4 + x : 0] *= f[x];
                    else sum = fmaf(st[4 * k4 + x], qv[x], sum);
                }
            }
            if (!LOCAL) {
                sum = glr_row16_sum(sum);
                if (g == 0 && live) orow[0] = sum;
                orow += (size_t)H * e;
            }
        }
        if (more) stage(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
    if (cb4 < ncb4) {
#pragma unroll
        for (int k = 0; k < RPL; ++k) S[(size_t)k * 64] = st[k];
    }
    if (LOCAL && cb16 == 0 && wave == 0 && cg == 0) {
        float* dr = decay + ((size_t)s * H + h) * DP + g * RPL;
#pragma unroll
        for (int k = 0; k < (LOCAL ? RPL : 1); ++k) dr[k] = dec[k];
    }
}

// Between the two passes over a prompt cut into `pieces` pieces per sequence: from the sequence's own state
// s_0 and every piece's local last state L_c and gate products D_c, the state each piece starts from,
// s_(c+1) = D_c s_c + L_c, written over L_c; the last one becomes the sequence's state.
// grid (sequences, heads * column blocks of 4), block 64.
__global__ __launch_bounds__(64) void glr_carry_kernel(float* __restrict__ state, size_t slot_stride,
                                                       const int* __restrict__ slots, float* __restrict__ piece_state,
                                                       size_t piece_stride, const float* __restrict__ decay, int pieces,
                                                       int H, int ncb4, int rpl) {
    const int b = blockIdx.x, hc = blockIdx.y, lane = threadIdx.x;
    const int slot = slots[b];
    if (slot < 0) return;
    const int h = hc / ncb4, dp = rpl * 16;
    for (int k = 0; k < rpl; ++k) {
        const size_t idx = ((size_t)hc * rpl + k) * 64 + lane;
        const int r = (lane & 15) * rpl + k;
        float sv = state[(size_t)slot * slot_stride + idx];
        for (int c = 0; c < pieces; ++c) {
            const size_t v = (size_t)b * pieces + c;
            const float local = piece_state[v * piece_stride + idx];
            piece_state[v * piece_stride + idx] = sv;
            sv = fmaf(decay[(v * H + h) * dp + r], sv, local);
        }
        state[(size_t)slot * slot_stride + idx] = sv;
    }
}

// Rows a lane holds for a head of d query channels: ceil(d / 16) rounded up to 4, 8, 16 or 32.
static inline int glr_rpl(int d) {
    const int r = (d + 15) / 16;
    return r <= 4 ? 4 : (r <= 8 ? 8 : (r <= 16 ? 16 : 32));
}
extern "C" int br_glr_rows_per_lane(int d) { return glr_rpl(d); }

template <bool LOCAL>
static int glr_scan_launch(const float* rows, const float* f_bias, const float* lower, float* o, float* state,
                           const int* cu_seqlens, const int* slots, int B, int H, int d, int e, int width,
                           size_t slot_stride, float* decay, hipStream_t s) {
    const int ncb4 = (e + 3) / 4, rpl = glr_rpl(d);
    if (H <= 0 || H > 65535 || d <= 0 || e <= 0 || d > 512 || (e + 15) / 16 > 65535 || width < 2 * H * d + H * e ||
        slot_stride < (size_t)H * ncb4 * rpl * 64 || (LOCAL && !decay))
        return BR_BAD_ARG;
    dim3 grid(B, H, (e + 15) / 16);
    // 16-byte loads where every row piece starts at a multiple of 16 bytes
    const bool v4 = d % 4 == 0 && width % 4 == 0 && ((uintptr_t)rows % 16) == 0;
#define GLR_SCAN(R, TC) do { \
        const size_t lds = (size_t)(4 * TC * R * 16 + 2 * TC * 16) * sizeof(float); \
        if (v4) glr_scan_kernel<R, TC, true, LOCAL><<<grid, 256, lds, s>>>(rows, f_bias, lower, o, state, cu_seqlens, slots, H, d, e, width, slot_stride, decay); \
        else glr_scan_kernel<R, TC, false, LOCAL><<<grid, 256, lds, s>>>(rows, f_bias, lower, o, state, cu_seqlens, slots, H, d, e, width, slot_stride, decay); \
    } while (0)
    if (rpl == 4) GLR_SCAN(4, 16);
    else if (rpl == 8) GLR_SCAN(8, 16);
    else if (rpl == 16) GLR_SCAN(16, 16);
    else GLR_SCAN(32, 8);
#undef GLR_SCAN
    return br_check_launch();
}

// `slot_stride`: floats from one slot's state to the next (at least H * ceil(e / 4) * rows per lane * 64).
extern "C" int br_glr_scan(const float* rows, const float* f_bias, const float* lower, float* o, float* state,
                           const int* cu_seqlens, const int* slots, int B, int H, int d, int e, int width,
                           size_t slot_stride, hipStream_t s) {
    if (B <= 0) return BR_OK;
    return glr_scan_launch<false>(rows, f_bias, lower, o, state, cu_seqlens, slots, B, H, d, e, width, slot_stride, nullptr, s);
}

// A step of long prompts with every sequence cut into `pieces` pieces that run side by side: the recurrence is
// linear in the state, so a piece can be walked from a zero state first (its last state L and the products D of
// its gates), the pieces' true first states follow from s_(c+1) = D_c s_c + L_c, and a second walk from those
// writes o.  Twice the arithmetic for `pieces` times the workgroups; results differ from the plain walk by the
// rounding of that one combination per piece.  `piece_cu` [B * pieces + 1] cuts the packed tokens (pieces of a
// sequence in order, empty ones allowed), `piece_slots` [B * pieces] is the piece's own number (or -1 for a
// padding sequence's), `piece_state` [B * pieces][state of a slot] and `decay` [B * pieces][H][16 * rows per lane]
// are scratch.
extern "C" int br_glr_scan_pieces(const float* rows, const float* f_bias, const float* lower, float* o, float* state,
                                  const int* slots, const int* piece_cu, const int* piece_slots, float* piece_state,
                                  float* decay, int B, int pieces, int H, int d, int e, int width, size_t slot_stride,
                                  hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (pieces <= 0 || (long long)B * pieces > 65535) return BR_BAD_ARG;
    const int ncb4 = (e + 3) / 4, rpl = glr_rpl(d);
    const size_t piece_stride = (size_t)H * ncb4 * rpl * 64;
    int rc = glr_scan_launch<true>(rows, f_bias, lower, o, piece_state, piece_cu, piece_slots, B * pieces, H, d, e, width,
                                   piece_stride, decay, s);
    if (rc != BR_OK) return rc;
    if ((long long)H * ncb4 > 65535) return BR_BAD_ARG;
    glr_carry_kernel<<<dim3(B, H * ncb4), 64, 0, s>>>(state, slot_stride, slots, piece_state, piece_stride, decay, pieces, H,
                                                      ncb4, rpl);
    rc = br_check_launch();
    if (rc != BR_OK) return rc;
    return glr_scan_launch<false>(rows, f_bias, lower, o, piece_state, piece_cu, piece_slots, B * pieces, H, d, e, width,
                                  piece_stride, nullptr, s);
}

// ------------------------------------------------------------------ head norm ------
// y[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * w.  16 lanes a (token, head) row, 16 rows a
// workgroup: a row of 128 channels is two 16-byte loads a lane, its sum of squares four moves between
// neighbouring lanes in a fixed order.
template <typename T, bool V4>
__global__ __launch_bounds__(256) void glr_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                            T* __restrict__ y, size_t n_rows, int e, float eps) {
    const size_t r = (size_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    const int l = threadIdx.x & 15;
    const bool on = r < n_rows;
    const float* orow = o + (on ? r : 0) * e;
    float ss = 0.f;
    if (V4) {
        for (int i = l; i < (e >> 2); i += 16) {
            const f32x4 v = on ? ((const f32x4*)orow)[i] : f32x4{0.f, 0.f, 0.f, 0.f};
            ss += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
        }
    } else {
        for (int i = l; i < e; i += 16) { const float v = on ? orow[i] : 0.f; ss += v * v; }
    }
    const float inv = 1.0f / sqrtf(glr_row16_sum(ss) / (float)e + eps);
    if (!on) return;
    T* yrow = y + r * e;
    if (V4) {
        for (int i = l; i < (e >> 2); i += 16) {
            const f32x4 v = ((const f32x4*)orow)[i];
            const f32x4 wv = w ? ((const f32x4*)w)[i] : f32x4{1.f, 1.f, 1.f, 1.f};
#pragma unroll
            for (int x = 0; x < 4; ++x) yrow[4 * i + x] = from_f32<T>(v[x] * inv * wv[x]);
        }
    } else {
        for (int i = l; i < e; i += 16) yrow[i] = from_f32<T>(orow[i] * inv * (w ? w[i] : 1.0f));
    }
}

extern "C" int br_glr_head_norm(const float* o, const float* w, void* y, int y_is_bf16, int T, int H, int e,
                                float eps, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (H <= 0 || e <= 0) return BR_BAD_ARG;
    const size_t n_rows = (size_t)T * H;
    const unsigned blocks = (unsigned)((n_rows + 15) / 16);
    const bool v4 = e % 4 == 0 && (((uintptr_t)o | (uintptr_t)w) % 16) == 0;
#define GLR_HN(TT, V) glr_head_norm_kernel<TT, V><<<blocks, 256, 0, s>>>(o, w, (TT*)y, n_rows, e, eps)
    if (y_is_bf16) { if (v4) GLR_HN(bf16, true); else GLR_HN(bf16, false); }
    else { if (v4) GLR_HN(float, true); else GLR_HN(float, false); }
#undef GLR_HN
    return br_check_launch();
}

// =====================================================================================
// A recurrence with a decay per key channel and a bonus for the current token: for a head with d key
// channels and e value channels,
//     o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,      S_t = diag(w_t) S_(t-1) + k_t v_t^T      (S is d x e, from zero)
// with the decay w_t = exp(-exp(z_t + w0)) in (0, 1) per channel made on the way into LDS from the float sums
// z_t of its projection, the receptance r, the key k and the bonus u (one number per head and key channel).
// Columns of S never meet, so the work is cut like `glr_scan_kernel`'s, the state lies in a slot as that
// kernel keeps it, and the walk is the same: TC tokens at a time through two LDS stages, the next chunk's rows
// in flight, a lane holding RPL rows of one column.  A token costs a lane 3 RPL / 4 reads of 16 bytes from LDS,
// one value, 4 RPL multiply-adds and the four moves that add the row groups' shares of o_t[c].
//
// rows [T, width] hold r | k | v | z at the column offsets 0, H d, 2 H d, 2 H d + H e (floats).
//
// LOCAL (the first pass over a long prompt cut into pieces, see `br_wkv_scan_pieces`): the state starts at zero,
// nothing is written to o, and beside the piece's last state the products of its decays go to `decay`
// ([sequences of the launch][head][16 RPL], in row order).
template <int RPL, int TC, bool V4, bool LOCAL>
__global__ __launch_bounds__(256) void wkv_scan_kernel(
    const float* __restrict__ rows, const float* __restrict__ w0, const float* __restrict__ bonus,
    float* __restrict__ o, float* __restrict__ state, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, int H, int d, int e, int width, size_t slot_stride, float* __restrict__ decay) {
    constexpr int DP = RPL * 16;
    constexpr int NL = TC * DP / 1024;
    extern __shared__ float lds[];
    float* wL = lds;                               // [2][TC][DP] decays
    float* kL = wL + 2 * TC * DP;                  // [2][TC][DP] keys
    float* rL = kL + 2 * TC * DP;                  // [2][TC][DP] receptances
    float* vL = rL + 2 * TC * DP;                  // [2][TC][16]
    const int s = blockIdx.x, h = blockIdx.y, cb16 = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cg = lane >> 4, g = lane & 15;
    const int cb4 = cb16 * 4 + wave, c = cb4 * 4 + cg;
    const int slot = slots[s];
    const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
    const bool live = c < e;
    if (slot < 0) {                                // padding: no state behind it; its rows of o are zero
        if (!LOCAL && g == 0 && live) for (int t = t0; t < t1; ++t) o[(size_t)t * H * e + h * e + c] = 0.f;
        return;
    }
    const int ncb4 = (e + 3) >> 2;
    float* S = state + (size_t)slot * slot_stride + (((size_t)h * ncb4 + cb4) * RPL) * 64 + lane;
    float st[RPL], ub[RPL];
#pragma unroll
    for (int k = 0; k < RPL; ++k) {
        st[k] = (!LOCAL && cb4 < ncb4) ? S[(size_t)k * 64] : 0.f;
        const int r = g * RPL + k;
        ub[k] = r < d ? bonus[h * d + r] : 0.f;
    }
    float dec[LOCAL ? RPL : 1];
#pragma unroll
    for (int k = 0; k < (LOCAL ? RPL : 1); ++k) dec[k] = 1.f;
    const int hd = H * d, he = H * e;
    int l_tt[NL], l_r4[NL];
    float b4[NL][4];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int idx = tid + 256 * i;
        l_tt[i] = idx / (DP / 4);
        l_r4[i] = (idx % (DP / 4)) * 4;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            const int r = l_r4[i] + x;
            b4[i][x] = r < d ? w0[h * d + r] : 0.f;
        }
    }
    const int v_tt = tid >> 4, v_c = cb16 * 16 + (tid & 15);
    float rr[NL][4], rk[NL][4], rz[NL][4], rv = 0.f;

    auto fetch = [&](int tc0) {
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const int t = tc0 + l_tt[i];
            const float* rp = rows + (size_t)t * width + h * d + l_r4[i];
            const float* zp = rows + (size_t)t * width + 2 * hd + he + h * d + l_r4[i];
            if (V4) {
                f32x4 a = {0.f, 0.f, 0.f, 0.f}, b = a, z = a;
                if (t < t1 && l_r4[i] < d) { a = *(const f32x4*)rp; b = *(const f32x4*)(rp + hd); z = *(const f32x4*)zp; }
#pragma unroll
                for (int x = 0; x < 4; ++x) { rr[i][x] = a[x]; rk[i][x] = b[x]; rz[i][x] = z[x]; }
            } else {
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const bool ok = t < t1 && l_r4[i] + x < d;
                    rr[i][x] = ok ? rp[x] : 0.f;
                    rk[i][x] = ok ? rp[hd + x] : 0.f;
                    rz[i][x] = ok ? zp[x] : 0.f;
                }
            }
        }
        const int t = tc0 + v_tt;
        rv = (v_tt < TC && t < t1 && v_c < e) ? rows[(size_t)t * width + 2 * hd + h * e + v_c] : 0.f;
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            f32x4 wo, ko, ro;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const bool real = l_r4[i] + x < d;
                wo[x] = real ? expf(-expf(rz[i][x] + b4[i][x])) : 1.f;
                ko[x] = real ? rk[i][x] : 0.f;
                ro[x] = real ? rr[i][x] : 0.f;
            }
            const size_t at = ((size_t)buf * TC + l_tt[i]) * DP + l_r4[i];
            *(f32x4*)(wL + at) = wo;
            *(f32x4*)(kL + at) = ko;
            *(f32x4*)(rL + at) = ro;
        }
        if (v_tt < TC) vL[(buf * TC + v_tt) * 16 + (tid & 15)] = rv;
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
        const float* wp = wL + (size_t)buf * TC * DP + g * RPL;
        const float* kp = kL + (size_t)buf * TC * DP + g * RPL;
        const float* rp = rL + (size_t)buf * TC * DP + g * RPL;
        const float* vp = vL + buf * TC * 16 + wave * 4 + cg;
#pragma unroll 2
        for (int tt = 0; tt < nt; ++tt) {
            const float vc = vp[tt * 16];
            float sum = 0.f;
#pragma unroll
            for (int k4 = 0; k4 < RPL / 4; ++k4) {
                const f32x4 wv = *(const f32x4*)(wp + (size_t)tt * DP + 4 * k4);
                const f32x4 kv4 = *(const f32x4*)(kp + (size_t)tt * DP + 4 * k4);
                f32x4 rv4 = {0.f, 0.f, 0.f, 0.f};
                if (!LOCAL) rv4 = *(const f32x4*)(rp + (size_t)tt * DP + 4 * k4);
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const float kv = kv4[x] * vc;
                    if (LOCAL) dec[LOCAL ? 4 * k4 + x : 0] *= wv[x];
                    else sum = fmaf(rv4[x], fmaf(ub[4 * k4 + x], kv, st[4 * k4 + x]), sum);
                    st[4 * k4 + x] = fmaf(wv[x], st[4 * k4 + x], kv);
                }
            }
            if (!LOCAL) {
                sum = glr_row16_sum(sum);
                if (g == 0 && live) orow[0] = sum;
                orow += he;
            }
        }
        if (more) stage(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
    if (cb4 < ncb4) {
#pragma unroll
        for (int k = 0; k < RPL; ++k) S[(size_t)k * 64] = st[k];
    }
    if (LOCAL && cb16 == 0 && wave == 0 && cg == 0) {
        float* dr = decay + ((size_t)s * H + h) * DP + g * RPL;
#pragma unroll
        for (int k = 0; k < (LOCAL ? RPL : 1); ++k) dr[k] = dec[k];
    }
}

// rows [T, width] float: r | k | v | z at 0, H d, 2 H d, 2 H d + H e; w0 and bonus float [H d]; o float [T, H e];
// `slot_stride`: floats from one slot's state to the next (at least H * ceil(e / 4) * rows per lane * 64).
template <bool LOCAL>
static int wkv_scan_launch(const float* rows, const float* w0, const float* bonus, float* o, float* state,
                           const int* cu_seqlens, const int* slots, int B, int H, int d, int e, int width,
                           size_t slot_stride, float* decay, hipStream_t s) {
    const int ncb4 = (e + 3) / 4, rpl = glr_rpl(d);
    if (H <= 0 || H > 65535 || d <= 0 || e <= 0 || d > 512 || (e + 15) / 16 > 65535 || width < 3 * H * d + H * e ||
        slot_stride < (size_t)H * ncb4 * rpl * 64 || !w0 || !bonus || (LOCAL && !decay))
        return BR_BAD_ARG;
    dim3 grid(B, H, (e + 15) / 16);
    const bool v4 = d % 4 == 0 && e % 4 == 0 && width % 4 == 0 && ((uintptr_t)rows % 16) == 0;
#define WKV_SCAN(R, TC) do { \
        const size_t lds = (size_t)(6 * TC * R * 16 + 2 * TC * 16) * sizeof(float); \
        if (v4) wkv_scan_kernel<R, TC, true, LOCAL><<<grid, 256, lds, s>>>(rows, w0, bonus, o, state, cu_seqlens, slots, H, d, e, width, slot_stride, decay); \
        else wkv_scan_kernel<R, TC, false, LOCAL><<<grid, 256, lds, s>>>(rows, w0, bonus, o, state, cu_seqlens, slots, H, d, e, width, slot_stride, decay); \
    } while (0)
    if (rpl == 4) WKV_SCAN(4, 16);
    else if (rpl == 8) WKV_SCAN(8, 16);
    else if (rpl == 16) WKV_SCAN(16, 8);
    else WKV_SCAN(32, 4);
#undef WKV_SCAN
    return br_check_launch();
}

extern "C" int br_wkv_scan(const float* rows, const float* w0, const float* bonus, float* o, float* state,
                           const int* cu_seqlens, const int* slots, int B, int H, int d, int e, int width,
                           size_t slot_stride, hipStream_t s) {
    if (B <= 0) return BR_OK;
    return wkv_scan_launch<false>(rows, w0, bonus, o, state, cu_seqlens, slots, B, H, d, e, width, slot_stride, nullptr, s);
}

// A step of long prompts with every sequence cut into `pieces` pieces that run side by side, as `br_glr_scan_pieces`
// does for its recurrence: a walk from zero (last state L, decay products D), s_(c+1) = D_c s_c + L_c by
// `glr_carry_kernel` (the bonus touches o only, never the state), a second walk from the true states that writes o.
extern "C" int br_wkv_scan_pieces(const float* rows, const float* w0, const float* bonus, float* o, float* state,
                                  const int* slots, const int* piece_cu, const int* piece_slots, float* piece_state,
                                  float* decay, int B, int pieces, int H, int d, int e, int width, size_t slot_stride,
                                  hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (pieces <= 0 || (long long)B * pieces > 65535) return BR_BAD_ARG;
    const int ncb4 = (e + 3) / 4, rpl = glr_rpl(d);
    const size_t piece_stride = (size_t)H * ncb4 * rpl * 64;
    int rc = wkv_scan_launch<true>(rows, w0, bonus, o, piece_state, piece_cu, piece_slots, B * pieces, H, d, e, width,
                                   piece_stride, decay, s);
    if (rc != BR_OK) return rc;
    if ((long long)H * ncb4 > 65535 || slot_stride < piece_stride) return BR_BAD_ARG;
    glr_carry_kernel<<<dim3(B, H * ncb4), 64, 0, s>>>(state, slot_stride, slots, piece_state, piece_stride, decay, pieces, H,
                                                      ncb4, rpl);
    rc = br_check_launch();
    if (rc != BR_OK) return rc;
    return wkv_scan_launch<false>(rows, w0, bonus, o, piece_state, piece_cu, piece_slots, B * pieces, H, d, e, width,
                                  piece_stride, nullptr, s);
}

// ------------------------------------------------------------- shifted mixes --------
// out[s][t][:] = h[t] + (h'[t] - h[t]) * mu[s] for `n_mix` mixing vectors mu [n_mix, W], with h' the row of the
// token before in the same sequence; before a step's first token it is the row the sequence's slot keeps
// (`kept`, float [W] at the start of what `kept + slot * slot_stride` points to; zeros in a new slot).  The
// differences are float; out has the rows' type.  A sequence that brings one token also leaves its row in the
// slot here; longer ones by `shift_keep_kernel` behind this one (their first token reads what the last replaces).
// grid (T, ceil(W / 256)).
template <typename T, int V>
__global__ __launch_bounds__(256) void shift_mix_kernel(const T* __restrict__ h, const float* __restrict__ mu,
                                                        T* __restrict__ out, float* __restrict__ kept, size_t slot_stride,
                                                        const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
                                                        const int* __restrict__ slots, int n_tok, int W, int n_mix) {
    // a thread brings V neighbouring columns (16 bytes of a row where the width allows it)
    typedef T vec_t __attribute__((ext_vector_type(V)));
    const int t = blockIdx.x, i = (blockIdx.y * 256 + threadIdx.x) * V;
    if (i >= W) return;
    const int b = seq_of_token[t], slot = slots[b];
    const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
    float cur[V], diff[V];
    if (V > 1) {
        const vec_t c = *(const vec_t*)(h + (size_t)t * W + i);
#pragma unroll
        for (int x = 0; x < V; ++x) cur[x] = to_f32<T>(c[x]);
    } else {
        cur[0] = to_f32<T>(h[(size_t)t * W + i]);
    }
    if (t > t0) {
        if (V > 1) {
            const vec_t p = *(const vec_t*)(h + (size_t)(t - 1) * W + i);
#pragma unroll
            for (int x = 0; x < V; ++x) diff[x] = to_f32<T>(p[x]) - cur[x];
        } else {
            diff[0] = to_f32<T>(h[(size_t)(t - 1) * W + i]) - cur[0];
        }
    } else {
#pragma unroll
        for (int x = 0; x < V; ++x) diff[x] = (slot >= 0 ? kept[(size_t)slot * slot_stride + i + x] : 0.f) - cur[x];
    }
    for (int s = 0; s < n_mix; ++s) {
        T* o = out + ((size_t)s * n_tok + t) * W + i;
        if (V > 1) {
            vec_t r;
#pragma unroll
            for (int x = 0; x < V; ++x) r[x] = from_f32<T>(fmaf(diff[x], mu[(size_t)s * W + i + x], cur[x]));
            *(vec_t*)o = r;
        } else {
            o[0] = from_f32<T>(fmaf(diff[0], mu[(size_t)s * W + i], cur[0]));
        }
    }
    if (slot >= 0 && t1 - t0 == 1) {
#pragma unroll
        for (int x = 0; x < V; ++x) kept[(size_t)slot * slot_stride + i + x] = cur[x];
    }
}

// The last row of every sequence that brought more than one token into its slot.  grid (B, ceil(W / 256)).
template <typename T>
__global__ __launch_bounds__(256) void shift_keep_kernel(const T* __restrict__ h, float* __restrict__ kept, size_t slot_stride,
                                                         const int* __restrict__ cu_seqlens, const int* __restrict__ slots, int W) {
    const int b = blockIdx.x, i = blockIdx.y * 256 + threadIdx.x;
    const int slot = slots[b];
    const int t0 = cu_seqlens[b], t1 = cu_seqlens[b + 1];
    if (i >= W || slot < 0 || t1 - t0 <= 1) return;
    kept[(size_t)slot * slot_stride + i] = to_f32<T>(h[(size_t)(t1 - 1) * W + i]);
}

extern "C" int br_shift_mix(const void* h, int is_bf16, const float* mu, void* out, float* kept, size_t slot_stride,
                            const int* seq_of_token, const int* cu_seqlens, const int* slots, int T, int B, int W, int n_mix,
                            int single_tokens, hipStream_t s) {
    if (T <= 0 || B <= 0) return BR_OK;
    if (W <= 0 || n_mix <= 0 || !kept || slot_stride < (size_t)W || (W + 255) / 256 > 65535 || B > 65535) return BR_BAD_ARG;
    dim3 keep_grid(B, (W + 255) / 256);
    // 16 bytes a thread where every row starts at a multiple of 16 bytes
    const bool vec = W % (is_bf16 ? 8 : 4) == 0 && (((uintptr_t)h | (uintptr_t)out) % 16) == 0;
    const int v = vec ? (is_bf16 ? 8 : 4) : 1;
    dim3 grid(T, (W / v + 255) / 256);
    if (is_bf16) {
        if (vec) shift_mix_kernel<bf16, 8><<<grid, 256, 0, s>>>((const bf16*)h, mu, (bf16*)out, kept, slot_stride, seq_of_token, cu_seqlens, slots, T, W, n_mix);
        else shift_mix_kernel<bf16, 1><<<grid, 256, 0, s>>>((const bf16*)h, mu, (bf16*)out, kept, slot_stride, seq_of_token, cu_seqlens, slots, T, W, n_mix);
    } else {
        if (vec) shift_mix_kernel<float, 4><<<grid, 256, 0, s>>>((const float*)h, mu, (float*)out, kept, slot_stride, seq_of_token, cu_seqlens, slots, T, W, n_mix);
        else shift_mix_kernel<float, 1><<<grid, 256, 0, s>>>((const float*)h, mu, (float*)out, kept, slot_stride, seq_of_token, cu_seqlens, slots, T, W, n_mix);
    }
    int rc = br_check_launch();
    if (rc != BR_OK || single_tokens) return rc;
    if (is_bf16) shift_keep_kernel<bf16><<<keep_grid, 256, 0, s>>>((const bf16*)h, kept, slot_stride, cu_seqlens, slots, W);
    else shift_keep_kernel<float><<<keep_grid, 256, 0, s>>>((const float*)h, kept, slot_stride, cu_seqlens, slots, W);
    return br_check_launch();
}

// ------------------------------------------------ head norm, weight and gate --------
// y[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * w[h, :] * silu(gate[t, h, :]): every head's output
// divided by its root mean square, a weight per head and channel, and a gate from the float sums of its
// projection (rows `gate_stride` floats apart; `gate_sigmoid`: sigmoid of the sums instead of silu).  16 lanes a
// (token, head) row as in `glr_head_norm_kernel`.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                             const float* __restrict__ gate, size_t gate_stride,
                                                             T* __restrict__ y, size_t n_rows, int H, int e, float eps,
                                                             int gate_sigmoid) {
    const size_t r = (size_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    const int l = threadIdx.x & 15;
    const bool on = r < n_rows;
    const float* orow = o + (on ? r : 0) * e;
    float ss = 0.f;
    for (int i = l; i < e; i += 16) { const float v = on ? orow[i] : 0.f; ss += v * v; }
    const float inv = 1.0f / sqrtf(glr_row16_sum(ss) / (float)e + eps);
    if (!on) return;
    const size_t t = r / H;
    const int hh = (int)(r - t * H);
    const float* grow = gate ? gate + t * gate_stride + (size_t)hh * e : nullptr;
    const float* wrow = w ? w + (size_t)hh * e : nullptr;
    T* yrow = y + r * e;
    for (int i = l; i < e; i += 16) {
        float v = orow[i] * inv;
        if (wrow) v *= wrow[i];
        if (grow) { const float z = grow[i]; v *= (gate_sigmoid ? 1.0f : z) / (1.0f + expf(-z)); }
        yrow[i] = from_f32<T>(v);
    }
}

// The same for rows of many channels (all heads normed together, say): a workgroup a (token, head) row.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_wide_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                                  const float* __restrict__ gate, size_t gate_stride,
                                                                  T* __restrict__ y, int H, int e, float eps, int gate_sigmoid) {
    __shared__ float scratch[16];
    const size_t r = blockIdx.x;
    const float* orow = o + r * e;
    float ss = 0.f;
    for (int i = threadIdx.x; i < e; i += 256) { const float v = orow[i]; ss = fmaf(v, v, ss); }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)e + eps);
    const size_t t = r / H;
    const int hh = (int)(r - t * H);
    const float* grow = gate ? gate + t * gate_stride + (size_t)hh * e : nullptr;
    const float* wrow = w ? w + (size_t)hh * e : nullptr;
    T* yrow = y + r * e;
    for (int i = threadIdx.x; i < e; i += 256) {
        float v = orow[i] * inv;
        if (wrow) v *= wrow[i];
        if (grow) { const float z = grow[i]; v *= (gate_sigmoid ? 1.0f : z) / (1.0f + expf(-z)); }
        yrow[i] = from_f32<T>(v);
    }
}

#define HNG_WIDE_FROM 512      // channels of a row from which a workgroup takes it

extern "C" int br_head_norm_gate(const float* o, const float* w, const float* gate, size_t gate_stride, void* y, int y_is_bf16,
                                 int T, int H, int e, float eps, int gate_sigmoid, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (H <= 0 || e <= 0 || (gate && gate_stride < (size_t)H * e)) return BR_BAD_ARG;
    const size_t n_rows = (size_t)T * H;
    if (e >= HNG_WIDE_FROM) {
        if (n_rows > 0x7fffffffULL) return BR_BAD_ARG;
        if (y_is_bf16) head_norm_gate_wide_kernel<bf16><<<(unsigned)n_rows, 256, 0, s>>>(o, w, gate, gate_stride, (bf16*)y, H, e, eps, gate_sigmoid);
        else head_norm_gate_wide_kernel<float><<<(unsigned)n_rows, 256, 0, s>>>(o, w, gate, gate_stride, (float*)y, H, e, eps, gate_sigmoid);
        return br_check_launch();
    }
    const unsigned blocks = (unsigned)((n_rows + 15) / 16);
    if (y_is_bf16) head_norm_gate_kernel<bf16><<<blocks, 256, 0, s>>>(o, w, gate, gate_stride, (bf16*)y, n_rows, H, e, eps, gate_sigmoid);
    else head_norm_gate_kernel<float><<<blocks, 256, 0, s>>>(o, w, gate, gate_stride, (float*)y, n_rows, H, e, eps, gate_sigmoid);
    return br_check_launch();
}

// y = tanh(x) elementwise, float sums in, the products' type out (the middle of a low-rank projection).
template <typename T>
__global__ __launch_bounds__(256) void tanh_kernel(const float* __restrict__ x, T* __restrict__ y, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = from_f32<T>(tanhf(x[i]));
}

extern "C" int br_tanh(const float* x, void* y, int y_is_bf16, size_t n, hipStream_t s) {
    if (n == 0) return BR_OK;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (y_is_bf16) tanh_kernel<bf16><<<blocks, 256, 0, s>>>(x, (bf16*)y, n);
    else tanh_kernel<float><<<blocks, 256, 0, s>>>(x, (float*)y, n);
    return br_check_launch();
}
