// Attention over a sliding window plus pooled blocks of the tokens that left it, over the
// paged cache, in float arithmetic for both storage types.
//
// A query at position p of its sequence sees the tokens lo..p, lo = max(0, p - size + 1),
// and one pooled key and value for every block b of `pool` tokens that lies wholly before
// the window: b * pool + pool - 1 <= p - size.  Pooled rows live in a cache unit of their
// own with one row per block (the means of the block's keys and of its values as the
// token cache holds them); both kinds of key share one softmax, which may carry a sink: a
// key of score 0 without a value, i.e. one added to the denominator.
//
// Three kernels: `prepare` (bias, per-head RMS norm of queries and keys, rotation of the
// first `rd` elements in (i, i + rd/2) pairs, value mixing with another layer's values,
// cache write), `pool` (the means of the blocks that the step completed) and `attend`.
// Keys and values of a page: keys [kv_head][token][dk] and, behind the keys of all heads, values
// transposed, [kv_head][dv][token]: the operand layout of the matrix-core kernel below (a lane reads
// 8 consecutive tokens of one value channel).
//
// The sums of `attend` run over the pages of the seen blocks and then over the pages of the window's
// tokens, so the order depends on (p, size, pool) only: whole prompts, portions and single tokens give
// the same bits.
//
// Further rules of what a query sees, each a parameter of the three attention kernels: `chunk` > 0 cuts the
// sequence into runs of `chunk` positions counted from 0 and a query sees no key of an earlier run (beside the
// window's rule; a window beyond any position leaves the runs alone); `keep` > 0 lets every query also see the
// sequence's first `keep` tokens, wherever its window begins.  The kept rows that lie before the window are
// walked first, like the pooled rows.  `softcap` > 0 bounds the scaled scores: s <- softcap tanh(s / softcap).
#include "common.h"

#define MAX_EPL 8   // head widths up to 64 * MAX_EPL

// The first position a query at p sees by its window and its run of `chunk` positions; both grow with p.
__device__ __forceinline__ int pwa_lo(int p, int size, int chunk) {
    int lo = p - size + 1;
    if (lo < 0) lo = 0;
    if (chunk > 0) {
        const int c = (p / chunk) * chunk;
        if (c > lo) lo = c;
    }
    return lo;
}

// ------------------------------------------------------------------- prepare -------
// qkv [T, width] float (the product's float sums: queries, keys, and the values from column `v_col0` on, which is
// nq*dk + nkv*dk when they have a projection of their own and nq*dk when the keys' sums, before their norm, are the
// values too), one wave per (token, head).  `q_every` > 0: the query is multiplied by
// 1 + q_coef ln(floor((p + 1) / q_every) + 1) at position p, behind its norm.
// vf_role: 0 none, 1 this layer's values are written to `v_first`, 2 values become
// (1 - lambda) v + lambda v_first.  Tokens of padding sequences (slot < 0) store nothing.
// `maps` > 1: every query and key head is `maps` vectors of dk side by side (several score maps over the same
// values), each normed and rotated by itself.  A key row of the cache is then maps * dk wide, and map m of a query
// head goes out as a row of that width with zeros outside its own dk elements, so that the attention kernels see
// nq * maps query heads over nkv kv heads whose scores are the maps' own.  `row_ss` [T, 2]: the sums of squares of
// the token's whole query and key projections (bias included); the norm then runs over the whole projection
// instead of a head, and `nw_stride` = dk gives every head norm weights of its own (0: one [dk] for all).
template <typename T>
__global__ __launch_bounds__(64) void pwa_prepare_kernel(
    const float* __restrict__ qkv, const float* __restrict__ bias, const float* __restrict__ qn_w,
    const float* __restrict__ kn_w, float eps, const float* __restrict__ cs, const float* __restrict__ sn,
    int rd, const int* __restrict__ pos, const int* __restrict__ seq_of_token,
    const int* __restrict__ slots, const int* __restrict__ block_table, int table_stride,
    T* __restrict__ q_out, T* __restrict__ storage, float* __restrict__ v_first,
    const float* __restrict__ lambda, int vf_role, int nq, int nkv, int dk, int dv, int page,
    int write_cache, int width, int v_col0, float q_coef, int q_every, int maps, const float* __restrict__ row_ss,
    int nw_stride, int pad_q) {
    extern __shared__ float row[];          // [max(dk, dv)]
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int nqs = nq * maps, nks = nkv * maps, kw = maps * dk;     // vectors of dk, and a key row's width
    const bool is_q = h < nqs, is_k = !is_q && h < nqs + nks;
    const int sub = is_q ? h : h - nqs;                              // which vector of the queries (keys)
    const int kvh = is_q ? 0 : (is_k ? sub / maps : h - nqs - nks);
    const int map = (is_q || is_k) ? sub % maps : 0;
    const int n = (is_q || is_k) ? dk : dv;
    const int col0 = is_q ? h * dk : (is_k ? nqs * dk + sub * dk : v_col0 + kvh * dv);
    const float* src = qkv + (size_t)t * width + col0;
    const int slot = slots[seq_of_token[t]];
    const int p = pos[t];
    T* dst = nullptr;
    if (is_q) {
        // `pad_q`: a query row as wide as a key row, with zeros where the other maps' keys lie; else dk wide
        T* qrow = q_out + ((size_t)t * nqs + h) * (pad_q ? kw : dk);
        dst = qrow + (pad_q ? map * dk : 0);
        for (int mm = 0; pad_q && mm < maps; ++mm)
            if (mm != map)
                for (int i = lane; i < dk; i += 64) qrow[mm * dk + i] = from_f32<T>(0.f);
    } else if (write_cache && slot >= 0) {
        const size_t page_elems = (size_t)nkv * page * (kw + dv);
        const int pg = block_table[(size_t)slot * table_stride + p / page];
        T* pb = storage + (size_t)pg * page_elems;
        dst = is_k ? pb + ((size_t)kvh * page + (p % page)) * kw + map * dk
                   : pb + (size_t)nkv * page * kw + (size_t)kvh * dv * page + (p % page);
    }
    const int dst_step = (is_q || is_k) ? 1 : page;      // values lie transposed: channel i of a token at i * page
    float v[MAX_EPL];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < MAX_EPL; ++j) {
        const int i = lane + 64 * j;
        v[j] = 0.f;
        if (i < n) {
            v[j] = src[i] + (bias ? bias[col0 + i] : 0.f);
            ss += v[j] * v[j];
        }
    }
    const bool qk = is_q || is_k;
    if (qk) {
        const float* nw = is_q ? qn_w : kn_w;
        if (nw) {
            const float inv = row_ss ? 1.0f / sqrtf(row_ss[2 * (size_t)t + (is_k ? 1 : 0)] / (float)((is_q ? nqs : nks) * dk) + eps)
                                     : 1.0f / sqrtf(wave_sum(ss) / (float)dk + eps);
            nw += (size_t)sub * nw_stride;
#pragma unroll
            for (int j = 0; j < MAX_EPL; ++j) {
                const int i = lane + 64 * j;
                if (i < n) v[j] = v[j] * inv * nw[i];
            }
        }
        if (is_q && q_every > 0) {          // the query's temperature: it grows with the logarithm of the position
            const float temp = 1.0f + q_coef * logf((float)((p + 1) / q_every) + 1.0f);
#pragma unroll
            for (int j = 0; j < MAX_EPL; ++j) v[j] *= temp;
        }
    }
    if (rd > 0) {                           // the barrier is met whatever the head
        const int half = rd >> 1;
        if (qk) {
#pragma unroll
            for (int j = 0; j < MAX_EPL; ++j) {
                const int i = lane + 64 * j;
                if (i < n) row[i] = v[j];
            }
        }
        __syncthreads();
        if (qk) {
#pragma unroll
            for (int j = 0; j < MAX_EPL; ++j) {
                const int i = lane + 64 * j;
                if (i < rd) {
                    const int f = i < half ? i : i - half;
                    const float c = cs[(size_t)t * half + f], s = sn[(size_t)t * half + f];
                    v[j] = i < half ? row[i] * c - row[i + half] * s : row[i] * c + row[i - half] * s;
                }
            }
        }
    }
    if (!qk && vf_role) {
        float* vf = v_first + (size_t)t * nkv * dv + (size_t)kvh * dv;
        const float lam = vf_role == 2 ? lambda[0] : 0.f;
#pragma unroll
        for (int j = 0; j < MAX_EPL; ++j) {
            const int i = lane + 64 * j;
            if (i < n) {
                if (vf_role == 1) vf[i] = v[j];
                else v[j] = (1.0f - lam) * v[j] + lam * vf[i];
            }
        }
    }
    if (dst) {
#pragma unroll
        for (int j = 0; j < MAX_EPL; ++j) {
            const int i = lane + 64 * j;
            if (i < n) dst[(size_t)i * dst_step] = from_f32<T>(v[j]);
        }
    }
}

// The values of a step of many tokens: a workgroup takes 64 packed tokens x 64 channels of one kv head through
// an LDS tile, so that the float sums are read in rows (bias, mixing and `v_first` as in `prepare`) and the
// transposed values are stored 64 neighbouring tokens of a channel at a time.  grid (ceil(T / 64), nkv,
// ceil(dv / 64)), block 256.
template <typename T>
__global__ __launch_bounds__(256) void pwa_values_kernel(
    const float* __restrict__ qkv, const float* __restrict__ bias, const int* __restrict__ pos,
    const int* __restrict__ seq_of_token, const int* __restrict__ slots, const int* __restrict__ block_table,
    int table_stride, T* __restrict__ storage, float* __restrict__ v_first, const float* __restrict__ lambda,
    int vf_role, int n_tokens, int nq, int nkv, int dk, int dv, int page, int width, int v_col0) {
    // `dk` is the width of a key row of the cache (all maps of a head)
    __shared__ float tile[64][65];
    const int t0 = blockIdx.x * 64, kvh = blockIdx.y, c0 = blockIdx.z * 64;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col0 = v_col0 + kvh * dv;
    const float lam = vf_role == 2 ? lambda[0] : 0.f;
    const int ch = c0 + lane;
    for (int r = 0; r < 16; ++r) {
        const int tt = wave + 4 * r, t = t0 + tt;
        float v = 0.f;
        if (t < n_tokens && ch < dv) {
            v = qkv[(size_t)t * width + col0 + ch] + (bias ? bias[col0 + ch] : 0.f);
            if (vf_role) {
                float* vf = v_first + (size_t)t * nkv * dv + (size_t)kvh * dv + ch;
                if (vf_role == 1) *vf = v;
                else v = (1.0f - lam) * v + lam * *vf;
            }
        }
        tile[tt][lane] = v;
    }
    __syncthreads();
    const int t = t0 + lane;
    if (t >= n_tokens) return;
    const int slot = slots[seq_of_token[t]];
    if (slot < 0) return;
    const int p = pos[t];
    const size_t page_elems = (size_t)nkv * page * (dk + dv);
    T* dst = storage + (size_t)block_table[(size_t)slot * table_stride + p / page] * page_elems + (size_t)nkv * page * dk +
             (size_t)kvh * dv * page + (p % page);
    for (int r = 0; r < 16; ++r) {
        const int cc = wave + 4 * r;
        if (c0 + cc < dv) dst[(size_t)(c0 + cc) * page] = from_f32<T>(tile[lane][cc]);
    }
}

// The sums of squares of a token's whole query projection and of its whole key projection (bias included), for a
// norm that runs over the projection instead of a head: out [T, 2].  grid (T), 256 threads, a fixed tree per row.
__global__ __launch_bounds__(256) void pwa_row_ss_kernel(const float* __restrict__ qkv, const float* __restrict__ bias,
                                                         float* __restrict__ out, int width, int nq_cols, int nk_cols) {
    __shared__ float scratch[16];
    const size_t t = blockIdx.x;
    const float* src = qkv + t * width;
    float sq = 0.f, sk = 0.f;
    if (((width | nq_cols | nk_cols) & 3) == 0 && (((uintptr_t)qkv | (uintptr_t)bias) & 15) == 0) {
        // 16 bytes a load; a thread's elements are added in their order, the threads' sums by a fixed tree
        const f32x4* s4 = (const f32x4*)src;
        const f32x4* b4 = (const f32x4*)bias;
        const int nq4 = nq_cols >> 2, n4 = (nq_cols + nk_cols) >> 2;
        for (int i = threadIdx.x; i < n4; i += 256) {
            f32x4 v = s4[i];
            if (b4) { const f32x4 b = b4[i]; v[0] += b[0]; v[1] += b[1]; v[2] += b[2]; v[3] += b[3]; }
            const float a = fmaf(v[3], v[3], fmaf(v[2], v[2], fmaf(v[1], v[1], v[0] * v[0])));
            if (i < nq4) sq += a; else sk += a;
        }
    } else {
        for (int i = threadIdx.x; i < nq_cols; i += 256) { const float v = src[i] + (bias ? bias[i] : 0.f); sq = fmaf(v, v, sq); }
        for (int i = nq_cols + threadIdx.x; i < nq_cols + nk_cols; i += 256) { const float v = src[i] + (bias ? bias[i] : 0.f); sk = fmaf(v, v, sk); }
    }
    sq = block_sum(sq, scratch);
    sk = block_sum(sk, scratch);
    if (threadIdx.x == 0) { out[2 * t] = sq; out[2 * t + 1] = sk; }
}

// `maps`, `row_ss` (scratch float [T, 2] when the norm runs over the whole projection, else null) and `nw_stride`:
// see the kernel.
extern "C" int br_pwa_prepare(const float* qkv, const float* bias, const float* qn_w, const float* kn_w, float eps,
                              const float* cs, const float* sn, int rd, const int* pos, const int* seq_of_token,
                              const int* slots, const int* block_table, int table_stride, void* q_out,
                              void* storage, int is_bf16, float* v_first, const float* lambda, int vf_role,
                              int T, int nq, int nkv, int dk, int dv, int page, int write_cache, int width, int v_from_k,
                              float q_coef, int q_every, int maps, float* row_ss, int nw_stride, int pad_q, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (maps <= 0 || (maps > 1 && v_from_k) || (nw_stride != 0 && nw_stride != dk)) return BR_BAD_ARG;
    const int nqs = nq * maps, nks = nkv * maps, kw = maps * dk;
    const int v_col0 = v_from_k ? nqs * dk : (nqs + nks) * dk;
    if (width < v_col0 + nkv * dv || (v_from_k && dv != dk) || (bias && v_from_k) || q_every < 0) return BR_BAD_ARG;
    if (nq <= 0 || nkv <= 0 || nq % nkv || dk <= 0 || dv <= 0 || kw > 64 * MAX_EPL || dv > 64 * MAX_EPL ||
        rd < 0 || rd > dk || (rd & 1) || page <= 0 || nqs + nks + nkv > 65535 || (rd > 0 && (!cs || !sn)) ||
        (vf_role && !v_first) || (vf_role == 2 && !lambda) || vf_role < 0 || vf_role > 2 || (row_ss && (!qn_w || !kn_w)))
        return BR_BAD_ARG;
    if (row_ss) {
        pwa_row_ss_kernel<<<T, 256, 0, s>>>(qkv, bias, row_ss, width, nqs * dk, nks * dk);
        const int rc0 = br_check_launch();
        if (rc0 != BR_OK) return rc0;
    }
    // steps of many tokens that store their values: the values by the tile kernel
    const bool tiled = T >= 256 && write_cache;
    dim3 grid(T, nqs + nks + (tiled ? 0 : nkv));
    const size_t lds = (size_t)(dk > dv ? dk : dv) * sizeof(float);
    if (is_bf16)
        pwa_prepare_kernel<bf16><<<grid, 64, lds, s>>>(qkv, bias, qn_w, kn_w, eps, cs, sn, rd, pos, seq_of_token, slots,
                                                       block_table, table_stride, (bf16*)q_out, (bf16*)storage, v_first,
                                                       lambda, vf_role, nq, nkv, dk, dv, page, write_cache, width, v_col0, q_coef, q_every,
                                                       maps, row_ss, nw_stride, pad_q);
    else
        pwa_prepare_kernel<float><<<grid, 64, lds, s>>>(qkv, bias, qn_w, kn_w, eps, cs, sn, rd, pos, seq_of_token, slots,
                                                        block_table, table_stride, (float*)q_out, (float*)storage,
                                                        v_first, lambda, vf_role, nq, nkv, dk, dv, page, write_cache, width, v_col0, q_coef, q_every,
                                                        maps, row_ss, nw_stride, pad_q);
    int rc = br_check_launch();
    if (rc != BR_OK || !tiled) return rc;
    dim3 vgrid((T + 63) / 64, nkv, (dv + 63) / 64);
    if (is_bf16)
        pwa_values_kernel<bf16><<<vgrid, 256, 0, s>>>(qkv, bias, pos, seq_of_token, slots, block_table, table_stride, (bf16*)storage,
                                                      v_first, lambda, vf_role, T, nq, nkv, kw, dv, page, width, v_col0);
    else
        pwa_values_kernel<float><<<vgrid, 256, 0, s>>>(qkv, bias, pos, seq_of_token, slots, block_table, table_stride, (float*)storage,
                                                       v_first, lambda, vf_role, T, nq, nkv, kw, dv, page, width, v_col0);
    return br_check_launch();
}

// ------------------------------------------------ two score maps into one head -----
// o[t, h, :] = (a1 - lambda a2) / sqrt(mean((a1 - lambda a2)^2) + eps) * scale, where a1 and a2 are the rows of the
// two maps of head h in `a` [T, nq, 2, dv] (what the attention kernels leave for 2 nq query heads).  `eps` < 0: no
// norm, o = (a1 - lambda a2) * scale.  A wave a (token, head) row, float arithmetic.  grid (ceil(T nq / 4)), 256.
template <typename T>
__global__ __launch_bounds__(256) void pwa_pair_combine_kernel(const T* __restrict__ a, T* __restrict__ o, size_t n_rows, int dv,
                                                               float lambda, float eps, float scale) {
    const size_t r = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (r >= n_rows) return;
    const T* a1 = a + r * 2 * dv;
    const T* a2 = a1 + dv;
    float v[MAX_EPL];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < MAX_EPL; ++j) {
        const int i = lane + 64 * j;
        v[j] = 0.f;
        if (i < dv) { v[j] = to_f32<T>(a1[i]) - lambda * to_f32<T>(a2[i]); ss = fmaf(v[j], v[j], ss); }
    }
    const float mul = eps < 0.f ? scale : scale / sqrtf(wave_sum(ss) / (float)dv + eps);
#pragma unroll
    for (int j = 0; j < MAX_EPL; ++j) {
        const int i = lane + 64 * j;
        if (i < dv) o[r * dv + i] = from_f32<T>(v[j] * mul);
    }
}

extern "C" int br_pwa_pair_combine(const void* a, void* o, int is_bf16, int T, int nq, int dv, float lambda, float eps,
                                   float scale, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (nq <= 0 || dv <= 0 || dv > 64 * MAX_EPL) return BR_BAD_ARG;
    const size_t n_rows = (size_t)T * nq;
    const unsigned blocks = (unsigned)((n_rows + 3) / 4);
    if (is_bf16) pwa_pair_combine_kernel<bf16><<<blocks, 256, 0, s>>>((const bf16*)a, (bf16*)o, n_rows, dv, lambda, eps, scale);
    else pwa_pair_combine_kernel<float><<<blocks, 256, 0, s>>>((const float*)a, (float*)o, n_rows, dv, lambda, eps, scale);
    return br_check_launch();
}

// ----------------------------------------------------------------- output gate -----
// o[t, h, i] <- o[t, h, i] * sigmoid(gate) * scale, with one gate number per element (gate row [nq * dv]) or one per
// head (gate row [nq]); the gate's rows are float sums `gate_stride` apart.  grid (T), 256 threads.
template <typename T>
__global__ __launch_bounds__(256) void pwa_gate_kernel(T* __restrict__ o, const float* __restrict__ gate, size_t gate_stride,
                                                       int nq, int dv, int per_head, float scale) {
    const size_t t = blockIdx.x;
    const int n = nq * dv;
    const float* grow = gate + t * gate_stride;
    T* orow = o + t * n;
    for (int i = threadIdx.x; i < n; i += 256) {
        const float z = grow[per_head ? i / dv : i];
        orow[i] = from_f32<T>(to_f32<T>(orow[i]) * (scale / (1.0f + expf(-z))));
    }
}

extern "C" int br_pwa_gate(void* o, int is_bf16, const float* gate, size_t gate_stride, int T, int nq, int dv, int per_head,
                           float scale, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (nq <= 0 || dv <= 0 || gate_stride < (size_t)(per_head ? nq : nq * dv)) return BR_BAD_ARG;
    if (is_bf16) pwa_gate_kernel<bf16><<<T, 256, 0, s>>>((bf16*)o, gate, gate_stride, nq, dv, per_head, scale);
    else pwa_gate_kernel<float><<<T, 256, 0, s>>>((float*)o, gate, gate_stride, nq, dv, per_head, scale);
    return br_check_launch();
}

// ---------------------------------------------------------------------- pool -------
// For sequence s with n new tokens ending at length L: the blocks b with
// start <= b * pool + pool - 1 < L (start = L - n) are complete after this step; their means go
// into row b of the pooled unit.  Block floor(start / pool) + blockIdx.y is this workgroup's;
// the grid's second size is max_new / pool + 1.
template <typename T>
__global__ __launch_bounds__(256) void pwa_pool_kernel(
    const T* __restrict__ storage, const int* __restrict__ block_table, int table_stride,
    T* __restrict__ pooled, const int* __restrict__ pooled_table, int pooled_stride,
    const int* __restrict__ cu_seqlens, const int* __restrict__ ctx_lens, const int* __restrict__ slots,
    int nkv, int dk, int dv, int page, int pool) {
    const int s = blockIdx.x, kvh = blockIdx.z;
    const int slot = slots[s];
    if (slot < 0) return;
    const int end = ctx_lens[s];
    const int start = end - (cu_seqlens[s + 1] - cu_seqlens[s]);
    const int b = start / pool + blockIdx.y;
    if ((long long)b * pool + pool > end) return;
    const size_t page_elems = (size_t)nkv * page * (dk + dv);
    const int* bt = block_table + (size_t)slot * table_stride;
    const int ppg = pooled_table[(size_t)slot * pooled_stride + b / page];
    T* pk = pooled + (size_t)ppg * page_elems + ((size_t)kvh * page + (b % page)) * dk;
    T* pv = pooled + (size_t)ppg * page_elems + (size_t)nkv * page * dk + (size_t)kvh * dv * page + (b % page);
    const float inv = 1.0f / (float)pool;
    for (int i = threadIdx.x; i < dk + dv; i += blockDim.x) {      // a channel a lane
        const bool key = i < dk;
        float acc = 0.f;
        // the rows are added in their order; eight are asked for at a time
        for (int r0 = 0; r0 < pool; r0 += 8) {
            float x[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int r = r0 + u;
                x[u] = 0.f;
                if (r < pool) {
                    const int j = b * pool + r;
                    const T* pb = storage + (size_t)bt[j / page] * page_elems;
                    x[u] = key ? to_f32<T>(pb[((size_t)kvh * page + (j % page)) * dk + i])
                               : to_f32<T>(pb[(size_t)nkv * page * dk + ((size_t)kvh * dv + (i - dk)) * page + (j % page)]);
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += x[u];
        }
        if (key) pk[i] = from_f32<T>(acc * inv);
        else pv[(size_t)(i - dk) * page] = from_f32<T>(acc * inv);
    }
}

extern "C" int br_pwa_pool(const void* storage, const int* block_table, int table_stride, void* pooled,
                           const int* pooled_table, int pooled_stride, const int* cu_seqlens, const int* ctx_lens,
                           const int* slots, int is_bf16, int B, int max_new, int nkv, int dk, int dv, int page,
                           int pool, hipStream_t s) {
    if (B <= 0) return BR_OK;
    if (nkv <= 0 || nkv > 65535 || dk <= 0 || dv <= 0 || page <= 0 || pool <= 0 || max_new <= 0) return BR_BAD_ARG;
    const int per_seq = max_new / pool + 1;
    if (per_seq > 65535) return BR_TOO_LARGE;
    dim3 grid(B, per_seq, nkv);
    const int threads = dk + dv > 128 ? 256 : (dk + dv > 64 ? 128 : 64);
    if (is_bf16)
        pwa_pool_kernel<bf16><<<grid, threads, 0, s>>>((const bf16*)storage, block_table, table_stride, (bf16*)pooled, pooled_table,
                                                  pooled_stride, cu_seqlens, ctx_lens, slots, nkv, dk, dv, page, pool);
    else
        pwa_pool_kernel<float><<<grid, threads, 0, s>>>((const float*)storage, block_table, table_stride, (float*)pooled,
                                                   pooled_table, pooled_stride, cu_seqlens, ctx_lens, slots, nkv, dk, dv,
                                                   page, pool);
    return br_check_launch();
}

// -------------------------------------------------------------------- attend -------
// One workgroup of four waves per (query token, query head), float arithmetic.  The query's keys come a
// page at a time: first the pages of the pooled unit that hold rows 0 .. seen - 1, then the token pages
// from the one that holds lo to the one that holds p; rows outside what the query sees are masked.  Page
// number n of that list is wave n % 4's.  A lane scores one row of the page (16 bytes a load where the
// width allows it), the wave takes an online-softmax step (m' = max(m, s), corr = exp(m - m'),
// l = l corr + sum w, acc = acc corr + w v), and in the second product a lane owns value channels and
// reads 8 neighbouring rows of a channel at a time from the transposed values.  The four waves' (m, l, acc)
// are merged in wave order at the end.  A sink starts wave 0 at m = 0, l = 1 instead of m = -inf, l = 0.
// Which page goes to which wave depends on (p, size, pool) only: whole prompts, portions and single
// tokens give the same bits.
template <typename T> struct pwa_vec;
template <> struct pwa_vec<float> { static constexpr int N = 4; typedef f32x4 type; };
template <> struct pwa_vec<bf16> { static constexpr int N = 8; typedef bf16x8 type; };

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void pwa_attend_kernel(
    const T* __restrict__ q, T* __restrict__ out, const int* __restrict__ pos,
    const int* __restrict__ seq_of_token, const int* __restrict__ slots,
    const int* __restrict__ block_table, int table_stride, const T* __restrict__ storage,
    const int* __restrict__ pooled_table, int pooled_stride, const T* __restrict__ pooled,
    int nq, int nkv, int dk, int dv, int page, int size, int pool, float scale, int sink, const float* __restrict__ sinks,
    int chunk, int keep, float softcap) {
    extern __shared__ float lds[];
    float* qs = lds;                         // [dk]
    float* ps = qs + dk;                     // [4][64]
    float* ml = ps + 256;                    // [4][2]
    float* accs = ml + 8;                    // [4][dv]
    constexpr int VN = pwa_vec<T>::N;
    typedef typename pwa_vec<T>::type vec_t;
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int kvh = h / (nq / nkv);
    T* o = out + ((size_t)t * nq + h) * dv;
    const int slot = slots[seq_of_token[t]];
    if (slot < 0) {
        for (int d = threadIdx.x; d < dv; d += 256) o[d] = from_f32<T>(0.f);
        return;
    }
    const T* qr = q + ((size_t)t * nq + h) * dk;
    for (int d = threadIdx.x; d < dk; d += 256) qs[d] = to_f32<T>(qr[d]);
    __syncthreads();
    const int p = pos[t];
    const int lo = pwa_lo(p, size, chunk);
    int seen = 0;
    if (pool > 0 && p - size - pool + 1 >= 0) seen = (p - size - pool + 1) / pool + 1;
    const int far_pages = (seen + page - 1) / page;
    const int kept = keep < lo ? keep : lo;                            // the first tokens that lie before the window
    const int kept_pages = (kept + page - 1) / page;
    const int first_page = lo / page, n_pages = far_pages + kept_pages + p / page - first_page + 1;
    const int* bt = block_table + (size_t)slot * table_stride;
    const int* pt = pooled_table ? pooled_table + (size_t)slot * pooled_stride : nullptr;
    const size_t page_elems = (size_t)nkv * page * (dk + dv);
    const size_t k_off = (size_t)kvh * page * dk, v_off = (size_t)nkv * page * dk + (size_t)kvh * dv * page;
    float* pw = ps + wave * 64;

    float m = (sink && wave == 0) ? (sinks ? sinks[h] : 0.f) : -INFINITY, l = (sink && wave == 0) ? 1.f : 0.f;
    float acc[MAX_EPL];
#pragma unroll
    for (int i = 0; i < MAX_EPL; ++i) acc[i] = 0.f;

    for (int n = wave; n < n_pages; n += 4) {
        const bool far = n < far_pages, early = !far && n < far_pages + kept_pages;
        const int pi = far ? n : (early ? n - far_pages : first_page + (n - far_pages - kept_pages));   // page index within its unit
        const T* base = far ? pooled + (size_t)pt[pi] * page_elems : storage + (size_t)bt[pi] * page_elems;
        const int row0 = pi * page;                                    // first row of the page
        const int first_ok = (far || early) ? 0 : lo, last_ok = far ? seen - 1 : (early ? kept - 1 : p);
        float s = -INFINITY;
        for (int j = lane; j < page; j += 64) {                       // pages of 64 rows: one row a lane
            const int key = row0 + j;
            if (key >= first_ok && key <= last_ok) {
                const T* kr = base + k_off + (size_t)j * dk;
                float dot = 0.f;
                if (VEC) {
                    for (int d = 0; d < dk; d += VN) {
                        const vec_t kv = *(const vec_t*)(kr + d);
#pragma unroll
                        for (int i = 0; i < VN; ++i) dot = fmaf(qs[d + i], to_f32<T>(kv[i]), dot);
                    }
                } else {
                    for (int d = 0; d < dk; ++d) dot = fmaf(qs[d], to_f32<T>(kr[d]), dot);
                }
                s = dot * scale;
                if (softcap > 0.f) s = softcap * tanhf(s / softcap);
            }
        }
        const float m_new = fmaxf(m, wave_max(s));
        if (m_new == -INFINITY) continue;                              // no row of this page is seen (wave-uniform)
        const float corr = expf(m - m_new);                            // exp(-inf) = 0 on a wave's first page
        const float w = expf(s - m_new);                               // 0 for masked rows
        l = l * corr + wave_sum(w);
        pw[lane] = w;
        m = m_new;
        // rows of this page that take part: [j_lo, j_hi)
        const int j_lo = first_ok > row0 ? first_ok - row0 : 0;
        const int j_hi = last_ok - row0 + 1 < page ? last_ok - row0 + 1 : page;
#pragma unroll
        for (int i = 0; i < MAX_EPL; ++i) {
            const int d = lane + 64 * i;
            if (d < dv) {
                const T* vr = base + v_off + (size_t)d * page;
                float a = acc[i] * corr;
                if (VEC) {
                    for (int j = (j_lo / VN) * VN; j < j_hi; j += VN) {
                        const vec_t vv = *(const vec_t*)(vr + j);
#pragma unroll
                        for (int e = 0; e < VN; ++e)
                            if (j + e >= j_lo && j + e < j_hi) a = fmaf(pw[j + e], to_f32<T>(vv[e]), a);
                    }
                } else {
                    for (int j = j_lo; j < j_hi; ++j) a = fmaf(pw[j], to_f32<T>(vr[j]), a);
                }
                acc[i] = a;
            }
        }
    }
    if (lane == 0) { ml[2 * wave] = m; ml[2 * wave + 1] = l; }
#pragma unroll
    for (int i = 0; i < MAX_EPL; ++i) {
        const int d = lane + 64 * i;
        if (d < dv) accs[wave * dv + d] = acc[i];
    }
    __syncthreads();
    float M = fmaxf(fmaxf(ml[0], ml[2]), fmaxf(ml[4], ml[6]));
    float L = 0.f, c4[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        c4[w] = ml[2 * w] == -INFINITY ? 0.f : expf(ml[2 * w] - M);
        L += ml[2 * w + 1] * c4[w];
    }
    for (int d = threadIdx.x; d < dv; d += 256) {
        float a = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) a += accs[w * dv + d] * c4[w];
        o[d] = from_f32<T>(a / L);
    }
}

extern "C" int br_pwa_attend(const void* q, void* out, int is_bf16, const int* pos, const int* seq_of_token,
                             const int* slots, const int* block_table, int table_stride, const void* storage,
                             const int* pooled_table, int pooled_stride, const void* pooled, int T, int nq, int nkv,
                             int dk, int dv, int page, int size, int pool, float scale, int sink, const float* __restrict__ sinks,
                             int chunk, int keep, float softcap, hipStream_t s) {
    if (T <= 0) return BR_OK;
    if (nq <= 0 || nkv <= 0 || nq % nkv || dk <= 0 || dv <= 0 || dk > 64 * MAX_EPL || dv > 64 * MAX_EPL || page != 64 ||
        size <= 0 || pool < 0 || nq > 65535 || (pool > 0 && (!pooled_table || !pooled)) || chunk < 0 || keep < 0 || !(softcap >= 0.f))
        return BR_BAD_ARG;
    dim3 grid(T, nq);
    const size_t lds = (size_t)(dk + 256 + 8 + 4 * dv) * sizeof(float);
    // 16-byte loads where every row starts at a multiple of 16 bytes
    const bool vec = is_bf16 ? dk % 8 == 0 : dk % 4 == 0;
#define PWA_ATT(TT, V) pwa_attend_kernel<TT, V><<<grid, 256, lds, s>>>((const TT*)q, (TT*)out, pos, seq_of_token, slots, block_table, \
        table_stride, (const TT*)storage, pooled_table, pooled_stride, (const TT*)pooled, nq, nkv, dk, dv, page, size, pool, scale, sink, sinks, \
        chunk, keep, softcap)
    if (is_bf16) { if (vec) PWA_ATT(bf16, true); else PWA_ATT(bf16, false); }
    else { if (vec) PWA_ATT(float, true); else PWA_ATT(float, false); }
#undef PWA_ATT
    return br_check_launch();
}

// ------------------------------------------------- prompts on the matrix cores -----
// bfloat16, pages of 64 rows, steps of several tokens per sequence.  grid = (row tiles of 128, nkv,
// sequences), block = 256.  A row is a (token, query head of the kv head's group) pair, row = token * G
// + head; each wave owns 32 rows and walks first the pooled rows, then the token rows its queries can
// see, 32 keys at a time.  Scores are computed transposed, S^T = K Q^T (v_mfma_f32_32x32x16_bf16, float
// sums), with the block's keys as the product's rows in a fixed permutation such that a lane's 16
// accumulators are 2 x 8 consecutive keys of its one query column: after the softmax step (float, base
// 2, the scale folded into the exponent) and rounding they are the B operand of O^T = V^T P^T as they
// stand, and V^T is read 16 contiguous bytes a lane from the transposed values.  NBK = ceil(dk / 32),
// NBV = ceil(dv / 32) (rounded up to a size that is compiled; surplus fragments are zero).
#define PWA_PAGE 64
#define PWA_LOG2E 1.4426950408889634f

__device__ __forceinline__ bf16x8 pwa_zero8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
    return z;
}
// 8 values V^T[channel][k .. k+7] of a page; rows at or beyond `limit` (not written yet) read as zero
__device__ __forceinline__ bf16x8 pwa_load_vt8(const bf16* __restrict__ vrow, int k, int limit) {
    bf16x8 v = *(const bf16x8*)(vrow + k);
    if (k + 8 > limit) {
#pragma unroll
        for (int i = 0; i < 8; ++i) if (k + i >= limit) v[i] = (bf16)0.f;
    }
    return v;
}
// Row c (0..31) of a score block stands for this key of the block; lane (column, g) then holds in
// acc[r] the key 16 (r / 8) + 8 g + r % 8.
__device__ __forceinline__ int pwa_key_of_row(int c) { return 16 * (c >> 4) + 8 * ((c >> 2) & 1) + 4 * ((c >> 3) & 1) + (c & 3); }

// One block of 32 keys (rows kb .. kb + 31 of a unit): `kblock` is the block's first key row (rows `ks` elements
// apart), `vblock` the first value channel at the block's first row (channels `vs` elements apart), in the cache
// or in LDS; rows of the block from `limit` on are not written and their values read as zero.  A key is seen by
// this lane's query if first_ok <= key <= last_ok.
template <int NBK, int NBV>
__device__ __forceinline__ void pwa_block(const bf16* __restrict__ kblock, int ks, const bf16* __restrict__ vblock, int vs,
                                          int kb, int limit, int first_ok, int last_ok, int dk, int dv, int c, int g,
                                          const bf16x8* qf, f32x16* acc_o, float& m, float& lsum, float scale2, float cap_in, float cap_out) {
    const bf16* krow = kblock + (size_t)pwa_key_of_row(c) * ks;
    f32x16 s_acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) s_acc[r] = 0.f;
#pragma unroll
    for (int s = 0; s < 2 * NBK; ++s) {
        const int d = s * 16 + 8 * g;
        const bf16x8 kf = (d < dk) ? *(const bf16x8*)(krow + d) : pwa_zero8();
        s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], s_acc, 0, 0, 0);
    }
    if (cap_out != 0.f) {
        // bounded scores: cap tanh(s scale / cap), tanh z = 1 - 2 / (exp(2 z) + 1); cap_in = 2 log2(e) scale / cap and
        // cap_out = cap / scale, so that the multiplication by scale2 below leaves the bounded score in base 2
#pragma unroll
        for (int r = 0; r < 16; ++r)
            s_acc[r] = cap_out * (1.0f - 2.0f * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(s_acc[r] * cap_in) + 1.0f));
    }
    float sv[16];
    float mx = -INFINITY;
    // the mask only where some lane's query does not see the whole block (the window's edges, the last pooled rows)
    const bool whole = __all(first_ok <= kb && kb + 31 <= last_ok);
    if (whole) {
#pragma unroll
        for (int r = 0; r < 16; ++r) { sv[r] = s_acc[r] * scale2; mx = fmaxf(mx, sv[r]); }
    } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = kb + 16 * (r >> 3) + 8 * g + (r & 7);
            sv[r] = (key >= first_ok && key <= last_ok) ? s_acc[r] * scale2 : -INFINITY;
            mx = fmaxf(mx, sv[r]);
        }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float corr = __builtin_amdgcn_exp2f(m - m_use);
    float psum = 0.f;
    bf16x8 p1, p2;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const float p = __builtin_amdgcn_exp2f(sv[r] - m_use);
        psum += p;
        if (r < 8) p1[r] = (bf16)p; else p2[r - 8] = (bf16)p;
    }
    lsum = lsum * corr + psum;
    // the sums so far are scaled only when some lane's maximum moved
    const bool moved = __any(m_new != m);
    m = m_new;
#pragma unroll
    for (int i = 0; i < NBV; ++i) {
        if (moved) {
#pragma unroll
            for (int r = 0; r < 16; ++r) acc_o[i][r] *= corr;
        }
        const int ch = i * 32 + c;
        bf16x8 v1 = pwa_zero8(), v2 = pwa_zero8();
        if (ch < dv) {
            const bf16* vrow = vblock + (size_t)ch * vs;
            v1 = pwa_load_vt8(vrow, 8 * g, limit);
            v2 = pwa_load_vt8(vrow, 16 + 8 * g, limit);
        }
        acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v1, p1, acc_o[i], 0, 0, 0);
        acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v2, p2, acc_o[i], 0, 0, 0);
    }
}

// Which tile of 128 rows a workgroup takes: the last tiles (most keys) first, so that the long workgroups start
// first; when all workgroups are resident at once, two to a compute unit (`pair`), the second half of the kv
// heads goes from short to long instead: the two workgroups that share a compute unit (their numbers lie half the
// grid apart) are then a long and a short one.
__device__ __forceinline__ int pwa_tile(int pair) {
    return (pair && ((blockIdx.y * 2 / gridDim.y) & 1)) ? blockIdx.x : gridDim.x - 1 - blockIdx.x;
}

// Two workgroups a compute unit (two waves a SIMD, so that one fills the other's waits) where the
// accumulators and operands leave room for it: keys and values up to 128 wide.
template <int NBK, int NBV>
__global__ __launch_bounds__(256, ((NBK <= 4 && NBV <= 4) ? 2 : 1)) void pwa_prefill_kernel(
    const bf16* __restrict__ q, bf16* __restrict__ out, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, const int* __restrict__ ctx_lens, const int* __restrict__ block_table,
    int table_stride, const bf16* __restrict__ storage, const int* __restrict__ pooled_table, int pooled_stride,
    const bf16* __restrict__ pooled, int nq, int nkv, int dk, int dv, int size, int pool, float scale, int sink, const float* __restrict__ sinks, int pair,
    int chunk, int keep, float softcap, int maps) {
    // `maps` > 1: blockIdx.y counts (kv head, map); a query row is dk wide and reads elements map * dk .. of the key
    // rows, which hold all maps side by side; nq counts the query rows of a token (heads x maps, the map innermost)
    const int b = blockIdx.z, kvh = blockIdx.y / maps, map = blockIdx.y % maps;
    const int slot = slots[b];
    const int t0 = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t0;
    const int G = nq / (nkv * maps), kw = maps * dk;
    const int rows_total = n_new * G;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row0 = pwa_tile(pair) * 128 + wave * 32;
    if (row0 >= rows_total) return;
    const int c = lane & 31, g = lane >> 5;
    const int row = row0 + c;
    const bool row_ok = row < rows_total;
    const int rr = row_ok ? row : rows_total - 1;
    const int tok = rr / G, head = (kvh * G + rr % G) * maps + map;
    bf16* orow = out + ((size_t)(t0 + tok) * nq + head) * dv;
    if (slot < 0) {       // padding: no cache behind it
        if (row_ok && g == 0) for (int d = 0; d < dv; ++d) orow[d] = (bf16)0.f;
        return;
    }
    const int ctx = ctx_lens[b], start = ctx - n_new;
    const int pq = start + tok;
    const int pq_min = start + row0 / G;
    const int last_row = (row0 + 31 < rows_total ? row0 + 31 : rows_total - 1);
    const int pq_max = start + last_row / G;

    const bf16* qrow = q + ((size_t)(t0 + tok) * nq + head) * dk;
    bf16x8 qf[2 * NBK];
#pragma unroll
    for (int s = 0; s < 2 * NBK; ++s) {
        const int d = s * 16 + 8 * g;
        qf[s] = (d < dk) ? *(const bf16x8*)(qrow + d) : pwa_zero8();
    }
    f32x16 acc_o[NBV];
#pragma unroll
    for (int i = 0; i < NBV; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[i][r] = 0.f;
    // the two lane halves of a query add their sums at the end: the sink's one goes to the first
    float m = sink ? (sinks ? sinks[head] * PWA_LOG2E : 0.f) : -INFINITY, lsum = (sink && g == 0) ? 1.f : 0.f;
    const float scale2 = scale * PWA_LOG2E;
    const bool capped = softcap > 0.f && scale != 0.f;
    const float cap_in = capped ? 2.0f * PWA_LOG2E * scale / softcap : 0.f, cap_out = capped ? softcap / scale : 0.f;
    const size_t page_elems = (size_t)nkv * PWA_PAGE * (kw + dv);
    const size_t k_off = (size_t)kvh * PWA_PAGE * kw + (size_t)map * dk, v_off = (size_t)nkv * PWA_PAGE * kw + (size_t)kvh * dv * PWA_PAGE;

    if (pool > 0) {
        // blocks wholly before the window: query p sees the pooled rows 0 .. seen(p) - 1
        const int far_max = pq_max - size - pool + 1, far = pq - size - pool + 1;
        const int seen_max = far_max >= 0 ? far_max / pool + 1 : 0;
        const int seen = (row_ok && far >= 0) ? far / pool + 1 : 0;
        const int written = ctx / pool;
        const int* pt = pooled_table + (size_t)slot * pooled_stride;
        for (int kb = 0; kb < seen_max; kb += 32) {
            const int kl = kb % PWA_PAGE;
            const bf16* pg = pooled + (size_t)pt[kb / PWA_PAGE] * page_elems;
            pwa_block<NBK, NBV>(pg + k_off + (size_t)kl * kw, kw, pg + v_off + kl, PWA_PAGE, kb, written - kb, 0, seen - 1, dk, dv, c, g,
                                qf, acc_o, m, lsum, scale2, cap_in, cap_out);
        }
    }
    const int* bt = block_table + (size_t)slot * table_stride;
    const int lo = pwa_lo(pq_min, size, chunk);
    const int first_ok = row_ok ? pwa_lo(pq, size, chunk) : 1, last_ok = row_ok ? pq : 0;
    if (keep > 0) {
        // the sequence's first tokens where they lie before a query's window
        const int lo_max = pwa_lo(pq_max, size, chunk);
        const int kept_max = keep < lo_max ? keep : lo_max, kept = row_ok ? (keep < first_ok ? keep : first_ok) : 0;
        for (int kb = 0; kb < kept_max; kb += 32) {
            const int kl = kb % PWA_PAGE;
            const bf16* pg = storage + (size_t)bt[kb / PWA_PAGE] * page_elems;
            pwa_block<NBK, NBV>(pg + k_off + (size_t)kl * kw, kw, pg + v_off + kl, PWA_PAGE, kb, ctx - kb, 0, kept - 1, dk, dv, c, g,
                                qf, acc_o, m, lsum, scale2, cap_in, cap_out);
        }
    }
    for (int kb = (lo / 32) * 32; kb <= pq_max; kb += 32) {
        const int kl = kb % PWA_PAGE;
        const bf16* pg = storage + (size_t)bt[kb / PWA_PAGE] * page_elems;
        pwa_block<NBK, NBV>(pg + k_off + (size_t)kl * kw, kw, pg + v_off + kl, PWA_PAGE, kb, ctx - kb, first_ok, last_ok, dk, dv, c, g,
                            qf, acc_o, m, lsum, scale2, cap_in, cap_out);
    }
    lsum += __shfl_xor(lsum, 32, 64);
    if (!row_ok) return;
    const float inv = lsum > 0.f ? 1.f / lsum : 0.f;
#pragma unroll
    for (int i = 0; i < NBV; ++i)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const int d = i * 32 + 8 * r4 + 4 * g;      // acc_o[i][4 r4 + e]: channel d + e
            if (d < dv) {
                bf16x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (bf16)(acc_o[i][4 * r4 + e] * inv);
                *(bf16x4*)(orow + d) = o;
            }
        }
}

// ------------------------------------------------ single tokens on the matrix cores -----
// Steps of one token per sequence, bfloat16: grid = (nkv, sequences), block = 64 PWA_DW (eight waves).  The G query heads of a kv
// head are the columns of the score blocks (G <= 32; the other columns idle), so the keys and values of a kv
// head are read once for all of its query heads.  The blocks of 32 keys the token sees (pooled rows first,
// then its window) are dealt to the waves in turn; each wave runs the online softmax over its blocks
// (wave 0 starts with the sink), and the waves' (m, l, O) are merged through LDS in wave order.  Eight waves:
// a wave's blocks follow one another with their loads' latencies in between (8 sequences that hold 1,024
// tokens: 31 us against 37 with four waves; 64 sequences: 102 against 92).
#define PWA_DW 8
template <int NBK, int NBV>
__global__ __launch_bounds__(64 * PWA_DW) void pwa_decode_kernel(
    const bf16* __restrict__ q, bf16* __restrict__ out, const int* __restrict__ slots,
    const int* __restrict__ ctx_lens, const int* __restrict__ block_table, int table_stride,
    const bf16* __restrict__ storage, const int* __restrict__ pooled_table, int pooled_stride,
    const bf16* __restrict__ pooled, int nq, int nkv, int dk, int dv, int size, int pool, float scale, int sink, const float* __restrict__ sinks, int cache_heads,
    int chunk, int keep, float softcap) {
    extern __shared__ float lds[];
    const int b = blockIdx.y, kvh = blockIdx.x;
    const int slot = slots[b];
    const int G = nq / nkv;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 31, g = lane >> 5;
    const bool row_ok = c < G;
    const int head = kvh * G + (row_ok ? c : G - 1);
    if (slot < 0) {       // padding: no cache behind it
        for (int i = threadIdx.x; i < G * dv; i += 64 * PWA_DW) out[((size_t)b * nq + kvh * G) * dv + i] = (bf16)0.f;
        return;
    }
    const int ctx = ctx_lens[b], pq = ctx - 1;
    const bf16* qrow = q + ((size_t)b * nq + head) * dk;
    bf16x8 qf[2 * NBK];
#pragma unroll
    for (int s = 0; s < 2 * NBK; ++s) {
        const int d = s * 16 + 8 * g;
        qf[s] = (d < dk) ? *(const bf16x8*)(qrow + d) : pwa_zero8();
    }
    f32x16 acc_o[NBV];
#pragma unroll
    for (int i = 0; i < NBV; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[i][r] = 0.f;
    float m = (sink && wave == 0) ? (sinks ? sinks[head] * PWA_LOG2E : 0.f) : -INFINITY, lsum = (sink && wave == 0 && g == 0) ? 1.f : 0.f;
    const float scale2 = scale * PWA_LOG2E;
    const bool capped = softcap > 0.f && scale != 0.f;
    const float cap_in = capped ? 2.0f * PWA_LOG2E * scale / softcap : 0.f, cap_out = capped ? softcap / scale : 0.f;
    // `nkv` blocks of query heads over `cache_heads` kv heads of the cache (more blocks than kv heads: several
    // workgroups read the same rows, each for its own query heads)
    const int ckv = (int)((long long)kvh * cache_heads / nkv);
    const size_t page_elems = (size_t)cache_heads * PWA_PAGE * (dk + dv);
    const size_t k_off = (size_t)ckv * PWA_PAGE * dk, v_off = (size_t)cache_heads * PWA_PAGE * dk + (size_t)ckv * dv * PWA_PAGE;
    int seen = 0;
    if (pool > 0 && pq - size - pool + 1 >= 0) seen = (pq - size - pool + 1) / pool + 1;
    const int far_blocks = (seen + 31) / 32;
    const int lo = pwa_lo(pq, size, chunk);
    const int kept = keep < lo ? keep : lo;                  // the first tokens that lie before the window
    const int kept_blocks = (kept + 31) / 32;
    const int kb0 = (lo / 32) * 32;
    const int n_blocks = far_blocks + kept_blocks + (pq - kb0) / 32 + 1;
    const int* bt = block_table + (size_t)slot * table_stride;
    const int* pt = pooled_table ? pooled_table + (size_t)slot * pooled_stride : nullptr;
    for (int n = wave; n < n_blocks; n += PWA_DW) {
        const bool far = n < far_blocks, early = !far && n < far_blocks + kept_blocks;
        const int kb = far ? n * 32 : (early ? (n - far_blocks) * 32 : kb0 + (n - far_blocks - kept_blocks) * 32);
        const int kl = kb % PWA_PAGE;
        const bf16* pg = far ? pooled + (size_t)pt[kb / PWA_PAGE] * page_elems : storage + (size_t)bt[kb / PWA_PAGE] * page_elems;
        const int limit = (far ? ctx / pool : ctx) - (kb - kl);
        const int first_ok = row_ok ? ((far || early) ? 0 : lo) : 1, last_ok = row_ok ? (far ? seen - 1 : (early ? kept - 1 : pq)) : 0;
        pwa_block<NBK, NBV>(pg + k_off + (size_t)kl * dk, dk, pg + v_off + kl, PWA_PAGE, kb, limit - kl, first_ok, last_ok, dk, dv, c, g,
                            qf, acc_o, m, lsum, scale2, cap_in, cap_out);
    }
    lsum += __shfl_xor(lsum, 32, 64);
    // merge: [wave][2 G lanes] of m and l, [wave][NBV * 16][2 G lanes] of O
    const int nl = 2 * G, li = g * G + c;
    float* mL = lds;                       // [PWA_DW][nl]
    float* lL = mL + PWA_DW * nl;          // [PWA_DW][nl]
    float* oL = lL + PWA_DW * nl;          // [PWA_DW][NBV * 16][nl]
    if (row_ok) {
        mL[wave * nl + li] = m;
        lL[wave * nl + li] = lsum;
#pragma unroll
        for (int i = 0; i < NBV; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oL[((size_t)wave * NBV * 16 + i * 16 + r) * nl + li] = acc_o[i][r];
    }
    __syncthreads();
    if (wave != 0 || !row_ok) return;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < PWA_DW; ++w) M = fmaxf(M, mL[w * nl + li]);
    float cw[PWA_DW], L = 0.f;
#pragma unroll
    for (int w = 0; w < PWA_DW; ++w) {
        const float mw = mL[w * nl + li];
        cw[w] = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - M);
        L += lL[w * nl + li] * cw[w];
    }
    const float inv = L > 0.f ? 1.f / L : 0.f;
    bf16* orow = out + ((size_t)b * nq + head) * dv;
#pragma unroll
    for (int i = 0; i < NBV; ++i)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const int d = i * 32 + 8 * r4 + 4 * g;
            if (d < dv) {
                bf16x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float a = 0.f;
#pragma unroll
                    for (int w = 0; w < PWA_DW; ++w) a += oL[((size_t)w * NBV * 16 + i * 16 + 4 * r4 + e) * nl + li] * cw[w];
                    o[e] = (bf16)(a * inv);
                }
                *(bf16x4*)(orow + d) = o;
            }
        }
}

template <int NBK>
static int pwa_decode_launch_v(int nbv, dim3 grid, size_t lds_of_nbv16, hipStream_t s, const bf16* q, bf16* out, const int* slots,
                               const int* ctx, const int* bt, int ts, const bf16* st, const int* pt, int ps, const bf16* pl,
                               int nq, int nkv, int dk, int dv, int size, int pool, float scale, int sink, const float* __restrict__ sinks, size_t head_lds, int cache_heads,
                               int chunk, int keep, float softcap) {
    // merges beyond 64 KB of LDS (many query heads to a kv head with wide values) are asked for once per kernel
#define PWA_GO(V) do { \
        auto kern = pwa_decode_kernel<NBK, V>; \
        const size_t lds = head_lds + lds_of_nbv16 * V; \
        static size_t have = 65536; \
        if (lds > have) { \
            if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) return BR_LAUNCH_FAILED; \
            have = lds; \
        } \
        kern<<<grid, 64 * PWA_DW, lds, s>>>(q, out, slots, ctx, bt, ts, st, pt, ps, pl, nq, nkv, dk, dv, size, pool, scale, sink, sinks, cache_heads, chunk, keep, softcap); \
    } while (0)
    if (nbv <= 1) PWA_GO(1);
    else if (nbv <= 2) PWA_GO(2);
    else if (nbv <= 3) PWA_GO(3);
    else if (nbv <= 4) PWA_GO(4);
    else PWA_GO(8);
#undef PWA_GO
    return br_check_launch();
}

// Bytes of LDS the merge of `pwa_decode_kernel` needs for these sizes (the launcher refuses more than 144 KB of a
// compute unit's 160).
static size_t pwa_decode_lds(int G, int dv) {
    const int nbv = (dv + 31) / 32, v = nbv <= 4 ? nbv : 8;
    return (size_t)(2 * PWA_DW * 2 * G + PWA_DW * v * 16 * 2 * G) * sizeof(float);
}
extern "C" int br_pwa_decode_takes(int nq, int nkv, int dk, int dv) {
    if (nq <= 0 || nkv <= 0 || nq % nkv || nq / nkv > 32 || dk <= 0 || dv <= 0 || dk > 256 || dv > 256 || dk % 8 || dv % 4) return 0;
    return pwa_decode_lds(nq / nkv, dv) <= 147456;
}

extern "C" int br_pwa_decode_bf16(const void* q, void* out, const int* slots, const int* ctx_lens, const int* block_table,
                                  int table_stride, const void* storage, const int* pooled_table, int pooled_stride,
                                  const void* pooled, int B, int nq, int nkv, int dk, int dv, int size, int pool, float scale,
                                  int sink, const float* __restrict__ sinks, int cache_heads, int chunk, int keep, float softcap, hipStream_t s) {
    // `nkv` counts the blocks of query heads a workgroup serves; the cache holds `cache_heads` kv heads (0: as many),
    // which `nkv` is a multiple of
    if (B <= 0) return BR_OK;
    if (cache_heads <= 0) cache_heads = nkv;
    if (!br_pwa_decode_takes(nq, nkv, dk, dv) || nkv > 65535 || B > 65535 || size <= 0 || pool < 0 || nkv % cache_heads ||
        (pool > 0 && (!pooled_table || !pooled)) || chunk < 0 || keep < 0 || !(softcap >= 0.f))
        return BR_BAD_ARG;
    const int G = nq / nkv;
    dim3 grid(nkv, B);
    const int nbk = (dk + 31) / 32, nbv = (dv + 31) / 32;
    const size_t head_lds = (size_t)2 * PWA_DW * 2 * G * sizeof(float), per_v = (size_t)PWA_DW * 16 * 2 * G * sizeof(float);
#define PWA_K(KK) pwa_decode_launch_v<KK>(nbv, grid, per_v, s, (const bf16*)q, (bf16*)out, slots, ctx_lens, block_table, table_stride, \
                                          (const bf16*)storage, pooled_table, pooled_stride, (const bf16*)pooled, nq, nkv, dk, dv, size, pool, scale, sink, sinks, head_lds, cache_heads, \
                                          chunk, keep, softcap)
    if (nbk <= 1) return PWA_K(1);
    if (nbk <= 2) return PWA_K(2);
    if (nbk <= 3) return PWA_K(3);
    if (nbk <= 4) return PWA_K(4);
    return PWA_K(8);
#undef PWA_K
}

// The same with a page's keys and values staged in LDS once for the workgroup's 128 rows: the pages its rows
// can see (pooled pages, then token pages) are walked by all four waves together; while a page is multiplied the
// next one is on its way from the cache into registers (16 bytes a lane and load, whole lines), and goes into
// the other LDS stage behind the page's one barrier.  Key rows lie PWA_PAD elements further apart than their
// width and value channels 64 + PWA_PAD apart, so that the 16-byte operand reads of a wave spread over the banks.
// A wave skips the blocks of a page that none of its own rows sees.
#define PWA_PAD 8

template <int NBK, int NBV>
__global__ __launch_bounds__(256, ((NBK <= 4 && NBV <= 4) ? 2 : 1)) void pwa_prefill_lds_kernel(
    const bf16* __restrict__ q, bf16* __restrict__ out, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, const int* __restrict__ ctx_lens, const int* __restrict__ block_table,
    int table_stride, const bf16* __restrict__ storage, const int* __restrict__ pooled_table, int pooled_stride,
    const bf16* __restrict__ pooled, int nq, int nkv, int dk, int dv, int size, int pool, float scale, int sink, const float* __restrict__ sinks, int pair,
    int chunk, int keep, float softcap, int maps) {
    extern __shared__ __attribute__((aligned(16))) unsigned char pwa_lds[];
    // `maps` > 1: as in `pwa_prefill_kernel`; a page's stage holds this map's part of the key rows only
    const int b = blockIdx.z, kvh = blockIdx.y / maps, map = blockIdx.y % maps;
    const int slot = slots[b];
    const int t0 = cu_seqlens[b], n_new = cu_seqlens[b + 1] - t0;
    const int G = nq / (nkv * maps), kw = maps * dk;
    const int rows_total = n_new * G;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wg_row0 = pwa_tile(pair) * 128;
    if (wg_row0 >= rows_total) return;                       // the whole workgroup
    const int row0 = wg_row0 + wave * 32;
    const bool wave_on = row0 < rows_total;
    const int c = lane & 31, g = lane >> 5;
    const int row = row0 + c;
    const bool row_ok = wave_on && row < rows_total;
    const int rr = row_ok ? row : rows_total - 1;
    const int tok = rr / G, head = (kvh * G + rr % G) * maps + map;
    bf16* orow = out + ((size_t)(t0 + tok) * nq + head) * dv;
    if (slot < 0) {       // padding: no cache behind it
        if (row_ok && g == 0) for (int d = 0; d < dv; ++d) orow[d] = (bf16)0.f;
        return;
    }
    const int ctx = ctx_lens[b], start = ctx - n_new;
    const int pq = start + tok;
    // positions of this wave's rows and of the workgroup's
    const int last_row = (row0 + 31 < rows_total ? row0 + 31 : rows_total - 1);
    const int pq_min = start + (wave_on ? row0 : wg_row0) / G, pq_max = start + (wave_on ? last_row : wg_row0) / G;
    const int wg_last = (wg_row0 + 127 < rows_total ? wg_row0 + 127 : rows_total - 1);
    const int wg_min = start + wg_row0 / G, wg_max = start + wg_last / G;

    const bf16* qrow = q + ((size_t)(t0 + tok) * nq + head) * dk;
    bf16x8 qf[2 * NBK];
#pragma unroll
    for (int s = 0; s < 2 * NBK; ++s) {
        const int d = s * 16 + 8 * g;
        qf[s] = (d < dk) ? *(const bf16x8*)(qrow + d) : pwa_zero8();
    }
    f32x16 acc_o[NBV];
#pragma unroll
    for (int i = 0; i < NBV; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[i][r] = 0.f;
    float m = sink ? (sinks ? sinks[head] * PWA_LOG2E : 0.f) : -INFINITY, lsum = (sink && g == 0) ? 1.f : 0.f;
    const float scale2 = scale * PWA_LOG2E;
    const bool capped = softcap > 0.f && scale != 0.f;
    const float cap_in = capped ? 2.0f * PWA_LOG2E * scale / softcap : 0.f, cap_out = capped ? softcap / scale : 0.f;
    const size_t page_elems = (size_t)nkv * PWA_PAGE * (kw + dv);
    const size_t k_off = (size_t)kvh * PWA_PAGE * kw + (size_t)map * dk, v_off = (size_t)nkv * PWA_PAGE * kw + (size_t)kvh * dv * PWA_PAGE;

    // what the wave's rows see, and the pages the workgroup walks
    auto seen_of = [&](int p) { const int far = p - size - pool + 1; return (pool > 0 && far >= 0) ? far / pool + 1 : 0; };
    const int seen = row_ok ? seen_of(pq) : 0, seen_wave = wave_on ? seen_of(pq_max) : 0;
    const int far_pages = (seen_of(wg_max) + PWA_PAGE - 1) / PWA_PAGE;
    const int wg_lo = pwa_lo(wg_min, size, chunk);
    const int lo_wave = pwa_lo(pq_min, size, chunk);
    const int first_page = wg_lo / PWA_PAGE;
    // the sequence's first `keep` tokens where they lie before a query's window: pages of their own in the walk
    auto kept_of = [&](int p) { const int l = pwa_lo(p, size, chunk); return keep < l ? keep : l; };
    const int kept = row_ok ? kept_of(pq) : 0, kept_wave = wave_on ? kept_of(pq_max) : 0;
    const int kept_pages = (kept_of(wg_max) + PWA_PAGE - 1) / PWA_PAGE;
    const int n_pages = far_pages + kept_pages + wg_max / PWA_PAGE - first_page + 1;
    const int written_far = pool > 0 ? ctx / pool : 0;
    const int first_ok = row_ok ? pwa_lo(pq, size, chunk) : 1, last_ok = row_ok ? pq : 0;
    const int* bt = block_table + (size_t)slot * table_stride;
    const int* pt = pooled_table ? pooled_table + (size_t)slot * pooled_stride : nullptr;

    const int ks = dk + PWA_PAD, vs = PWA_PAGE + PWA_PAD;
    const size_t stage_elems = (size_t)PWA_PAGE * ks + (size_t)dv * vs;
    bf16* stage0 = (bf16*)pwa_lds;
    // a page's keys are PAGE * dk / 8 pieces of 16 bytes, its values dv * 8: each thread brings up to NBK + NBV of each
    const int k_pieces = PWA_PAGE * dk / 8, v_pieces = dv * 8;
    bf16x8 rk[NBK], rv[NBV];
    // where a thread's pieces of the keys lie in a page: row (piece / pieces a row) of the page's key rows, kw apart
    int k_src[NBK];
#pragma unroll
    for (int i = 0; i < NBK; ++i) {
        const int piece = threadIdx.x + 256 * i, per = dk / 8;
        k_src[i] = (piece / per) * kw + (piece % per) * 8;
    }
    auto page_of = [&](int n) -> const bf16* {
        if (n < far_pages) return pooled + (size_t)pt[n] * page_elems;
        if (n < far_pages + kept_pages) return storage + (size_t)bt[n - far_pages] * page_elems;
        return storage + (size_t)bt[first_page + (n - far_pages - kept_pages)] * page_elems;
    };
    auto fetch = [&](int n) {
        const bf16* pg = page_of(n);
#pragma unroll
        for (int i = 0; i < NBK; ++i) {
            const int piece = threadIdx.x + 256 * i;
            rk[i] = piece < k_pieces ? *(const bf16x8*)(pg + k_off + k_src[i]) : pwa_zero8();
        }
#pragma unroll
        for (int i = 0; i < NBV; ++i) {
            const int piece = threadIdx.x + 256 * i;
            rv[i] = piece < v_pieces ? *(const bf16x8*)(pg + v_off + (size_t)piece * 8) : pwa_zero8();
        }
    };
    auto put = [&](int buf) {
        bf16* st = stage0 + (size_t)buf * stage_elems;
        const int per_row = dk / 8;
#pragma unroll
        for (int i = 0; i < NBK; ++i) {
            const int piece = threadIdx.x + 256 * i;
            if (piece < k_pieces) *(bf16x8*)(st + (size_t)(piece / per_row) * ks + (piece % per_row) * 8) = rk[i];
        }
        bf16* sv = st + (size_t)PWA_PAGE * ks;
#pragma unroll
        for (int i = 0; i < NBV; ++i) {
            const int piece = threadIdx.x + 256 * i;
            if (piece < v_pieces) *(bf16x8*)(sv + (size_t)(piece >> 3) * vs + (piece & 7) * 8) = rv[i];
        }
    };
    fetch(0);
    put(0);
    __syncthreads();
    for (int n = 0; n < n_pages; ++n) {
        const int buf = n & 1;
        if (n + 1 < n_pages) fetch(n + 1);
        const bf16* st = stage0 + (size_t)buf * stage_elems;
        const bf16* sv = st + (size_t)PWA_PAGE * ks;
        const bool far = n < far_pages, early = !far && n < far_pages + kept_pages;
        const int page_row0 = (far ? n : (early ? n - far_pages : first_page + (n - far_pages - kept_pages))) * PWA_PAGE;
#pragma unroll
        for (int hb = 0; hb < 2; ++hb) {
            const int kb = page_row0 + 32 * hb;
            const bool mine = wave_on && (far ? kb < seen_wave : (early ? kb < kept_wave : (kb + 31 >= lo_wave && kb <= pq_max)));     // wave-uniform
            if (mine)
                pwa_block<NBK, NBV>(st + (size_t)(32 * hb) * ks, ks, sv + 32 * hb, vs, kb, (far ? written_far : ctx) - kb,
                                    (far || early) ? 0 : first_ok, far ? seen - 1 : (early ? kept - 1 : last_ok), dk, dv, c, g, qf, acc_o, m, lsum,
                                    scale2, cap_in, cap_out);
        }
        if (n + 1 < n_pages) put(buf ^ 1);
        __syncthreads();
    }
    lsum += __shfl_xor(lsum, 32, 64);
    if (!row_ok) return;
    const float inv = lsum > 0.f ? 1.f / lsum : 0.f;
#pragma unroll
    for (int i = 0; i < NBV; ++i)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
            const int d = i * 32 + 8 * r4 + 4 * g;
            if (d < dv) {
                bf16x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (bf16)(acc_o[i][4 * r4 + e] * inv);
                *(bf16x4*)(orow + d) = o;
            }
        }
}

template <int NBK>
static int pwa_prefill_launch_v(int nbv, dim3 grid, hipStream_t s, const bf16* q, bf16* out, const int* cu, const int* slots,
                                const int* ctx, const int* bt, int ts, const bf16* st, const int* pt, int ps, const bf16* pl,
                                int nq, int nkv, int dk, int dv, int size, int pool, float scale, int sink, const float* __restrict__ sinks,
                                int chunk, int keep, float softcap, int maps) {
    // steps that fill a workgroup's 128 rows stage the pages in LDS (key widths in steps of 8 and value widths in steps
    // of 8 that the kernel's pieces cover); shorter ones read their operands straight from the cache
    const int cus = br_device_cus();
    const int pair = cus > 0 && (long long)grid.x * grid.y * grid.z <= 2LL * cus;
    const bool staged = (long long)grid.x * 128 >= 256 && dv % 8 == 0 && dk <= NBK * 32 && dk * 8 <= NBK * 256;
    const size_t lds = (size_t)2 * ((size_t)PWA_PAGE * (dk + PWA_PAD) + (size_t)dv * (PWA_PAGE + PWA_PAD)) * sizeof(bf16);
#define PWA_GO(V) do { \
        if (staged && dv * 8 <= V * 256) { \
            auto kern = pwa_prefill_lds_kernel<NBK, V>; \
            static size_t have = 0; \
            if (lds > have) { \
                if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) return BR_LAUNCH_FAILED; \
                have = lds; \
            } \
            kern<<<grid, 256, lds, s>>>(q, out, cu, slots, ctx, bt, ts, st, pt, ps, pl, nq, nkv, dk, dv, size, pool, scale, sink, sinks, pair, chunk, keep, softcap, maps); \
        } else pwa_prefill_kernel<NBK, V><<<grid, 256, 0, s>>>(q, out, cu, slots, ctx, bt, ts, st, pt, ps, pl, nq, nkv, dk, dv, size, pool, scale, sink, sinks, pair, chunk, keep, softcap, maps); \
    } while (0)
    if (nbv <= 1) PWA_GO(1);
    else if (nbv <= 2) PWA_GO(2);
    else if (nbv <= 3) PWA_GO(3);
    else if (nbv <= 4) PWA_GO(4);
    else PWA_GO(8);
#undef PWA_GO
    return br_check_launch();
}

// Takes bfloat16, widths of keys in steps of 8 and of values in steps of 4, each up to 256.  `maps` > 1: `nq` counts a
// token's query rows (heads x maps, the map innermost), each dk wide; the cache's key rows are maps * dk wide, and
// every (kv head, map) is a workgroup column of its own, so no product is spent on another map's key elements.
extern "C" int br_pwa_prefill_bf16(const void* q, void* out, const int* cu_seqlens, const int* slots, const int* ctx_lens,
                                   const int* block_table, int table_stride, const void* storage, const int* pooled_table,
                                   int pooled_stride, const void* pooled, int B, int max_new, int nq, int nkv, int dk, int dv,
                                   int size, int pool, float scale, int sink, const float* __restrict__ sinks, int chunk, int keep,
                                   float softcap, int maps, hipStream_t s) {
    if (B <= 0 || max_new <= 0) return BR_OK;
    if (maps <= 0 || nq <= 0 || nkv <= 0 || nq % (nkv * maps) || nkv * maps > 65535 || B > 65535 || dk <= 0 || dv <= 0 || dk > 256 || dv > 256 || dk % 8 ||
        dv % 4 || size <= 0 || pool < 0 || (pool > 0 && (!pooled_table || !pooled)) || chunk < 0 || keep < 0 || !(softcap >= 0.f))
        return BR_BAD_ARG;
    const int G = nq / (nkv * maps);
    dim3 grid((unsigned)(((size_t)max_new * G + 127) / 128), nkv * maps, B);
    const int nbk = (dk + 31) / 32, nbv = (dv + 31) / 32;
#define PWA_K(KK) pwa_prefill_launch_v<KK>(nbv, grid, s, (const bf16*)q, (bf16*)out, cu_seqlens, slots, ctx_lens, block_table, table_stride, \
                                           (const bf16*)storage, pooled_table, pooled_stride, (const bf16*)pooled, nq, nkv, dk, dv, size, pool, scale, sink, sinks, \
                                           chunk, keep, softcap, maps)
    if (nbk <= 1) return PWA_K(1);
    if (nbk <= 2) return PWA_K(2);
    if (nbk <= 3) return PWA_K(3);
    if (nbk <= 4) return PWA_K(4);
    return PWA_K(8);
#undef PWA_K
}
