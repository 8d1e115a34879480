// Token mixers over a RAGGED step: the tokens of all rows of a step lie back to back, row b owning
// tokens [row_start[b], row_start[b] + row_len[b]) that continue its sequence at position row_ctx[b]
// (a prompt's portion of any length beside single decoded tokens).  What a sequence carries between
// steps lives either in pages of a key/value pool (block_table) or in its state slot (row_slot);
// a row with row_ctx == 0 starts from zero state whatever its slot held before.
//
//   conv_silu / conv_state_update  short causal convolution per channel with its tail kept per slot
//   conv_taps                      the same convolution without bias or activation, optionally added to its
//                                  input (y = u + conv(u)); output in fp32 and / or the activation type
//   conv_qkv_store                 the convolution over the q | k | v columns of one projection: queries to a
//                                  buffer, keys and values straight into their pages
//   softplus_decay                 step sizes and decays of a selective state-space head
//   scan_outer                     S_t = decay_t S_(t-1) + gain_t k_t v_t^T,  o_t = S_t^T q_t (+ skip_h v_t)
//                                  (state-space duality heads and fixed-decay retention heads alike)
//   scan_gated                     S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T,  o_t = S_t^T q_t: a forget gate per
//                                  state row that also scales what is written (no key)
//   gate_lower_bound               q = silu(q), f = l + (1 - l) sigmoid(f + b) in place, ahead of scan_gated
//   rotary_pairs                   rotate-half rotation of the first `rot` dimensions of each head
//   gated_group_norm               unit-RMS per group with a SiLU gate before or after it
//   qk_unitnorm_store              per-head unit-RMS of queries and keys, keys/values into their pages
//   qk_rotary_store                biases on queries and keys, rotation of both over the first `rot` dimensions
//                                  of a head (adjacent pairs or halves); the rotated key into the key page and the
//                                  key as projected into the value page (attention whose values are its keys)
//   window_attn                    softmax attention over the last `window` positions (and, where asked for, the
//                                  sequence's first `keep_first` positions) with a per-head linear distance
//                                  penalty and / or a per-head sink in the denominator
// All of it in fp32; the activation type (bf16 or fp32) only concerns what goes to a projection or
// into the key/value pages.
#include "common.h"

namespace mv {

template <bool F32> struct ActS;
template <> struct ActS<true> {
    typedef float T;
    static __device__ __forceinline__ float ld(const float* p) { return *p; }
    static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct ActS<false> {
    typedef uint16_t T;
    static __device__ __forceinline__ float ld(const uint16_t* p) { return bf16_bits_to_f32(*p); }
    static __device__ __forceinline__ void st(uint16_t* p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }
};

__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + expf(-v)); }

struct StepRows {
    const int* tok_row;    // [T] row of each token
    const int* tok_pos;    // [T] position of each token in its sequence
    const int* row_start;  // [B]
    const int* row_len;    // [B]
    const int* row_ctx;    // [B] tokens the sequence held before this step
    const int* row_slot;   // [B] state slot
};

constexpr int kMaxTaps = 16;

__global__ __launch_bounds__(256) void conv_silu_kernel(const float* in, int64_t ldi, const float* state,
                                                        const float* w, const float* bias, float* out, int64_t ldo,
                                                        StepRows r, int T, int C, int taps) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)T * C) return;
    const int t = (int)(i / C), c = (int)(i % C);
    const int b = r.tok_row[t];
    const int rel = t - r.row_start[b];
    const bool carried = r.row_ctx[b] > 0;
    const float* st = state + ((int64_t)r.row_slot[b] * (taps - 1)) * C + c;
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int src = rel - (taps - 1) + j;  // portion-relative index of the input under tap j
        float v;
        if (src >= 0) v = in[(int64_t)(t - (taps - 1) + j) * ldi + c];
        else v = carried ? st[(int64_t)(src + taps - 1) * C] : 0.f;
        acc = fmaf(w[(int64_t)c * taps + j], v, acc);
    }
    out[(int64_t)t * ldo + c] = silu_f(acc);
}

__global__ __launch_bounds__(256) void conv_state_update_kernel(const float* in, int64_t ldi, float* state,
                                                                StepRows r, int B, int C, int taps) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)B * C) return;
    const int b = (int)(i / C), c = (int)(i % C);
    const int keep = taps - 1, len = r.row_len[b], start = r.row_start[b];
    const bool carried = r.row_ctx[b] > 0;
    float* st = state + ((int64_t)r.row_slot[b] * keep) * C + c;
    float old[kMaxTaps];
    for (int s = 0; s < keep; ++s) old[s] = carried ? st[(int64_t)s * C] : 0.f;
    for (int s = 0; s < keep; ++s) {
        const int rel = len - keep + s;
        st[(int64_t)s * C] = rel >= 0 ? in[(int64_t)(start + rel) * ldi + c] : old[s + len];
    }
}

__global__ __launch_bounds__(256) void softplus_decay_kernel(const float* raw, int64_t ld, const float* dt_bias,
                                                             const float* a_log, float* gain, float* decay,
                                                             float* log_decay, int T, int H) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= T * H) return;
    const int t = i / H, h = i % H;
    const float v = raw[(int64_t)t * ld + h] + dt_bias[h];
    const float dt = fmaxf(v, 0.f) + log1pf(expf(-fabsf(v)));  // log(1 + e^v), no clamp
    gain[i] = dt;
    const float ld_ = -expf(a_log[h]) * dt;
    decay[i] = expf(ld_);
    if (log_decay) log_decay[i] = ld_;
}

struct ScanArgs {
    const float *q, *k, *v, *decay, *gain, *skip;
    int64_t ldq, ldk, ldv, ld_decay, ld_gain, ldo;
    int q_div, k_div;
    float* state;
    float* out;
    StepRows r;
    int H, n, p, pt;
    int max_len;   // rows longer than this belong to the chunked form (0: every row is taken)
    // chunk mode (ch_start != NULL): blockIdx.z is a chunk of a long row, run from a zero state; what it
    // leaves goes to ds[chunk][head] instead of the slot
    const int *ch_start, *ch_len;
    float* ds;
};

// GATED: `decay` holds a forget gate per (token, head, state row) and the key is one minus it.
template <int MAXN, bool GATED = false>
__global__ __launch_bounds__(256) void scan_outer_kernel(ScanArgs a) {
    __shared__ float part[2][256];
    const int b = blockIdx.z, h = blockIdx.y, tid = threadIdx.x;
    const int PT = a.pt, NS = 256 / PT;
    const int cl = tid % PT, ng = tid / PT, c = blockIdx.x * PT + cl;
    const bool vc = c < a.p;
    const int npt = (a.n + NS - 1) / NS, n0 = ng * npt;
    const bool chunk = a.ch_start != nullptr;
    const int len = chunk ? a.ch_len[b] : a.r.row_len[b], start = chunk ? a.ch_start[b] : a.r.row_start[b];
    if (!chunk && a.max_len > 0 && len > a.max_len) return;   // the whole workgroup
    const bool carried = !chunk && a.r.row_ctx[b] > 0;
    float* sp = (chunk ? a.ds + (((int64_t)b * a.H + h) * a.n + n0) * a.p
                       : a.state + (((int64_t)a.r.row_slot[b] * a.H + h) * a.n + n0) * a.p) + c;
    float S[MAXN];
#pragma unroll
    for (int i = 0; i < MAXN; ++i) S[i] = (carried && vc && i < npt && n0 + i < a.n) ? sp[(int64_t)i * a.p] : 0.f;
    for (int t = 0; t < len; ++t) {
        const int64_t tok = start + t;
        const float vv = vc ? a.v[tok * a.ldv + (int64_t)h * a.p + c] : 0.f;
        const float* qp = a.q + tok * a.ldq + (int64_t)(h / a.q_div) * a.n + n0;
        float o = 0.f;
        if (GATED) {
            const float* fp = a.decay + tok * a.ld_decay + (int64_t)h * a.n + n0;
#pragma unroll
            for (int i = 0; i < MAXN; ++i) {
                if (i < npt && n0 + i < a.n) {
                    const float f = fp[i];
                    S[i] = fmaf(1.0f - f, vv, f * S[i]);
                    o = fmaf(S[i], qp[i], o);
                }
            }
        } else {
            const float dec = a.decay[tok * a.ld_decay + h];
            const float g = a.gain ? a.gain[tok * a.ld_gain + h] : 1.0f;
            const float gv = g * vv;
            const float* kp = a.k + tok * a.ldk + (int64_t)(h / a.k_div) * a.n + n0;
#pragma unroll
            for (int i = 0; i < MAXN; ++i) {
                if (i < npt && n0 + i < a.n) {
                    S[i] = fmaf(kp[i], gv, dec * S[i]);
                    o = fmaf(S[i], qp[i], o);
                }
            }
        }
        part[t & 1][tid] = o;
        __syncthreads();
        if (ng == 0 && vc) {
            float tot = 0.f;
            for (int j = 0; j < NS; ++j) tot += part[t & 1][j * PT + cl];
            if (a.skip) tot = fmaf(a.skip[h], vv, tot);
            a.out[tok * a.ldo + (int64_t)h * a.p + c] = tot;
        }
    }
    if (vc) {
#pragma unroll
        for (int i = 0; i < MAXN; ++i)
            if (i < npt && n0 + i < a.n) sp[(int64_t)i * a.p] = S[i];
    }
}

// ---- the same recurrence in chunks of 64 tokens, for rows long enough to pay for three launches ----
// Within a chunk that starts from state S0, with L_t the running sum of log decay over the chunk:
//   o_t = exp(L_t) S0^T q_t + sum_{s<=t} exp(L_t - L_s) gain_s (q_t . k_s) v_s
//   S_end = exp(L_end) S0 + sum_s exp(L_end - L_s) gain_s k_s v_s^T
// intra:  per (chunk, head)  the second term of o, the sum of S_end (dS) and exp(L_end), L_t kept
// carry:  per (row, head)    S0 of every chunk in turn (left where dS was), the row's final state
// inter:  per (chunk, head)  o_t += exp(L_t) S0^T q_t (+ skip_h v_t)
// fp32 throughout; differs from the token-by-token form by the order of the sums only.
constexpr int kCh = 64;

struct ChunkArgs {
    const float *q, *k, *v, *log_decay, *gain, *skip;
    int64_t ldq, ldk, ldv, ld_ld, ld_gain, ldo;
    int q_div, k_div;
    float* state;
    float* out;
    float* ds;     // [chunks, H, n, p]
    float* lsum;   // [tokens, H]  L_t
    float* atot;   // [chunks, H]  exp(L_end)
    const int *ch_start, *ch_len, *row_ch0, *row_nch;
    StepRows r;
    int H, n, p;
    int hb;   // heads of one group a workgroup takes in turn (they share q, k and the products q . k)
};

// All three products of a chunk run on v_mfma_f32_16x16x4_f32 (true fp32): operand A lane (r, g) = A[r][g],
// operand B lane (r, g) = B[g][r], result lane (r, g) = C[4 g + j][r] (r = lane % 16, g = lane / 16).
#define MV_MFMA4(acc, a_, b_) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a_, b_, acc, 0, 0, 0)

__global__ __launch_bounds__(256) void scan_chunk_intra_kernel(ChunkArgs a) {
    extern __shared__ float lds[];
    const int ch = blockIdx.x, tid = threadIdx.x;
    const int wv = tid >> 6, r = tid & 15, qd = (tid & 63) >> 4;
    const int n = a.n, p = a.p, n4 = (n + 3) & ~3, sn = n4 + 1, sp = p + 1;
    float* qs = lds;
    float* ks = qs + kCh * sn;
    float* vs = ks + kCh * sn;
    float* Ls = vs + kCh * sp;
    float* gs = Ls + kCh;
    float* ws = gs + kCh;
    const int start = a.ch_start[ch], len = a.ch_len[ch];
    // a.hb heads of one group per workgroup: they share q and k, staged once, and the products q_t . k_s
    const int h_first = blockIdx.y * a.hb;
    for (int i = tid; i < kCh * n4; i += 256) {
        const int t = i / n4, j = i % n4;
        const bool ok = t < len && j < n;
        qs[t * sn + j] = ok ? a.q[(int64_t)(start + t) * a.ldq + (int64_t)(h_first / a.q_div) * n + j] : 0.f;
        ks[t * sn + j] = ok ? a.k[(int64_t)(start + t) * a.ldk + (int64_t)(h_first / a.k_div) * n + j] : 0.f;
    }
    __syncthreads();
    // wave wv owns the tokens t = 16 wv + r.  P0[nt][j] = q_t . k_s, s = 16 nt + 4 qd + j, s-tiles above the
    // diagonal stay zero: A = k rows of the s-tile, B = q rows of the wave's tokens, summed over the state index
    const int t0 = 16 * wv, t = t0 + r;
    f32x4_t P0[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) P0[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    for (int j0 = 0; j0 < n4; j0 += 4) {
        const float bq = qs[t * sn + j0 + qd];
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
            if (nt <= wv) MV_MFMA4(P0[nt], ks[(16 * nt + r) * sn + j0 + qd], bq);
    }
    for (int hh = 0; hh < a.hb; ++hh) {
        const int h = h_first + hh;
        __syncthreads();   // the head before is done with vs, Ls, gs, ws
        for (int i = tid; i < kCh * p; i += 256) {
            const int tt = i / p, c = i % p;
            vs[tt * sp + c] = tt < len ? a.v[(int64_t)(start + tt) * a.ldv + (int64_t)h * p + c] : 0.f;
        }
        if (tid < kCh) {   // one wave: inclusive running sum of the log decays
            float l = 0.f, g = 0.f;
            if (tid < len) {
                l = fmaxf(a.log_decay[(int64_t)(start + tid) * a.ld_ld + h], -80.f);
                g = a.gain ? a.gain[(int64_t)(start + tid) * a.ld_gain + h] : 1.f;
            }
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const float up = __shfl_up(l, o, 64);
                if (tid >= o) l += up;
            }
            Ls[tid] = l;
            gs[tid] = g;
            if (tid < len) a.lsum[(int64_t)(start + tid) * a.H + h] = l;
            const float lend = __shfl(l, len - 1, 64);
            ws[tid] = expf(lend - l) * g;        // weight of token s in the state the chunk ends with
            if (tid == 0) a.atot[(int64_t)ch * a.H + h] = expf(lend);
        }
        __syncthreads();
        f32x4_t P[4];
        {
            const float Lt = Ls[t];
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int s_ = 16 * nt + 4 * qd + j;
                    P[nt][j] = (s_ <= t) ? P0[nt][j] * expf(Lt - Ls[s_]) * gs[s_] : 0.f;
                }
        }
        // o[t][c] = sum_s P[t][s] v[s][c]: A = v^T (columns c), B = P straight from the registers
        for (int c0 = 0; c0 < p; c0 += 64) {
            f32x4_t o[4];
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) o[ct] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
                if (nt > wv) continue;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float* vrow = vs + (16 * nt + 4 * qd + j) * sp;
#pragma unroll
                    for (int ct = 0; ct < 4; ++ct) {
                        const int c = c0 + 16 * ct + r;
                        MV_MFMA4(o[ct], c < p ? vrow[c] : 0.f, P[nt][j]);
                    }
                }
            }
            if (t < len) {
#pragma unroll
                for (int ct = 0; ct < 4; ++ct)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int c = c0 + 16 * ct + 4 * qd + j;
                        if (c < p) a.out[(int64_t)(start + t) * a.ldo + (int64_t)h * p + c] = o[ct][j];
                    }
            }
        }
        // dS[j][c] = sum_s (k[s][j] ws[s]) v[s][c]: A = k^T weighted as it is read, B = v, over the tokens
        float* dsp = a.ds + ((int64_t)ch * a.H + h) * n * p;
        for (int jt = wv; jt * 16 < n; jt += 4) {
            const int ja = 16 * jt + r;
            for (int c0 = 0; c0 < p; c0 += 64) {
                f32x4_t dd[4];
#pragma unroll
                for (int ct = 0; ct < 4; ++ct) dd[ct] = f32x4_t{0.f, 0.f, 0.f, 0.f};
                for (int s0 = 0; s0 < kCh; s0 += 4) {
                    const float ak = ja < n4 ? ks[(s0 + qd) * sn + ja] * ws[s0 + qd] : 0.f;
                    const float* vrow = vs + (s0 + qd) * sp;
#pragma unroll
                    for (int ct = 0; ct < 4; ++ct) {
                        const int c = c0 + 16 * ct + r;
                        MV_MFMA4(dd[ct], ak, c < p ? vrow[c] : 0.f);
                    }
                }
#pragma unroll
                for (int ct = 0; ct < 4; ++ct)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int jj = 16 * jt + 4 * qd + j, c = c0 + 16 * ct + r;
                        if (jj < n && c < p) dsp[(int64_t)jj * p + c] = dd[ct][j];
                    }
            }
        }
    }
}

__global__ __launch_bounds__(256) void scan_chunk_carry_kernel(ChunkArgs a) {
    const int b = blockIdx.z, h = blockIdx.y;
    const int np = a.n * a.p, e = blockIdx.x * 256 + threadIdx.x;
    const int nch = a.row_nch[b];
    if (nch == 0 || e >= np) return;
    float* sp = a.state + ((int64_t)a.r.row_slot[b] * a.H + h) * np + e;
    float S = a.r.row_ctx[b] > 0 ? *sp : 0.f;
    const int c0 = a.row_ch0[b];
    for (int c = c0; c < c0 + nch; ++c) {
        float* d = a.ds + ((int64_t)c * a.H + h) * np + e;
        const float add = *d;
        *d = S;                                   // the state this chunk starts from
        S = fmaf(a.atot[(int64_t)c * a.H + h], S, add);
    }
    *sp = S;
}

__global__ __launch_bounds__(256) void scan_chunk_inter_kernel(ChunkArgs a) {
    extern __shared__ float lds[];
    const int ch = blockIdx.x, tid = threadIdx.x;
    const int wv = tid >> 6, r = tid & 15, qd = (tid & 63) >> 4;
    const int n = a.n, p = a.p, n4 = (n + 3) & ~3, sn = n4 + 1, sp = p + 1;
    float* qs = lds;
    float* Ss = qs + kCh * sn;
    const int start = a.ch_start[ch], len = a.ch_len[ch];
    const int h_first = blockIdx.y * a.hb;
    for (int i = tid; i < kCh * n4; i += 256) {
        const int t = i / n4, j = i % n4;
        qs[t * sn + j] =
            (t < len && j < n) ? a.q[(int64_t)(start + t) * a.ldq + (int64_t)(h_first / a.q_div) * n + j] : 0.f;
    }
    const int t = 16 * wv + r;
    for (int hh = 0; hh < a.hb; ++hh) {
        const int h = h_first + hh;
        __syncthreads();
        const float* dsp = a.ds + ((int64_t)ch * a.H + h) * n * p;
        for (int i = tid; i < n4 * p; i += 256) Ss[(i / p) * sp + i % p] = i < n * p ? dsp[i] : 0.f;
        __syncthreads();
        // o[t][c] += exp(L_t) sum_j q[t][j] S0[j][c]: A = S0^T (columns c), B = q rows of the wave's tokens
        const float sk = a.skip ? a.skip[h] : 0.f;
        const float w = t < len ? expf(a.lsum[(int64_t)(start + t) * a.H + h]) : 0.f;
        for (int c0 = 0; c0 < p; c0 += 64) {
            f32x4_t o[4];
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) o[ct] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            for (int j0 = 0; j0 < n4; j0 += 4) {
                const float bq = qs[t * sn + j0 + qd];
                const float* srow = Ss + (j0 + qd) * sp;
#pragma unroll
                for (int ct = 0; ct < 4; ++ct) {
                    const int c = c0 + 16 * ct + r;
                    MV_MFMA4(o[ct], c < p ? srow[c] : 0.f, bq);
                }
            }
            if (t < len) {
#pragma unroll
                for (int ct = 0; ct < 4; ++ct)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int c = c0 + 16 * ct + 4 * qd + j;
                        if (c >= p) continue;
                        float* op = a.out + (int64_t)(start + t) * a.ldo + (int64_t)h * p + c;
                        float res = fmaf(w, o[ct][j], *op);
                        if (a.skip) res = fmaf(sk, a.v[(int64_t)(start + t) * a.ldv + (int64_t)h * p + c], res);
                        *op = res;
                    }
            }
        }
    }
}

// ---- the gated recurrence in chunks of 64 tokens ----
// Within a chunk that starts from state S0, with P_t[i] the product of the gates f_s[i] over the chunk's tokens
// s <= t:  o_t = (local run from a zero state)_t + sum_i q_t[i] P_t[i] S0[i][:],  S_end = diag(P_end) S0 + local.
//   gate_cumprod   P_t for every token of every chunk
//   scan_outer_kernel in chunk mode: the local runs, all chunks side by side
//   gated_carry    per (row, head): the state each chunk starts from, in turn (left where the local sum was),
//                  and the row's final state
//   gated_inter    o_t += (q_t * P_t) S0, a [64 x n] . [n x p] product per (chunk, head) in fp32
// Products of gates, no logarithms: a gate of exactly zero or one is exact, long decays underflow to zero as
// the token-by-token run does.
__global__ __launch_bounds__(256) void gate_cumprod_kernel(const float* f, int64_t ldf, float* cum, int64_t ldc,
                                                           const int* ch_start, const int* ch_len, int width) {
    const int ch = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= width) return;
    const int start = ch_start[ch], len = ch_len[ch];
    float pr = 1.0f;
    for (int t = 0; t < len; ++t) {
        pr *= f[(int64_t)(start + t) * ldf + c];
        cum[(int64_t)(start + t) * ldc + c] = pr;
    }
}

struct GatedChunkArgs {
    const float* q;
    const float* cum;
    int64_t ldq, ldc, ldo;
    float* state;
    float* out;
    float* ds;
    const int *ch_start, *ch_len, *row_ch0, *row_nch, *row_ctx, *row_slot;
    int H, n, p;
};

__global__ __launch_bounds__(256) void gated_carry_kernel(GatedChunkArgs a) {
    const int b = blockIdx.z, h = blockIdx.y;
    const int np = a.n * a.p, e = blockIdx.x * 256 + threadIdx.x;
    const int nch = a.row_nch[b];
    if (nch == 0 || e >= np) return;
    const int i = e / a.p;
    float* sp = a.state + ((int64_t)a.row_slot[b] * a.H + h) * np + e;
    float S = a.row_ctx[b] > 0 ? *sp : 0.f;
    const int c0 = a.row_ch0[b];
    for (int c = c0; c < c0 + nch; ++c) {
        float* d = a.ds + ((int64_t)c * a.H + h) * np + e;
        const float add = *d;
        *d = S;                                   // the state this chunk starts from
        const int last = a.ch_start[c] + a.ch_len[c] - 1;
        S = fmaf(a.cum[(int64_t)last * a.ldc + (int64_t)h * a.n + i], S, add);
    }
    *sp = S;
}

// one workgroup per (chunk, head, 64 value columns): thread (ty, tx) owns 4 tokens x 4 columns
__global__ __launch_bounds__(256) void gated_inter_kernel(GatedChunkArgs a) {
    __shared__ float as[16][kCh + 4];
    __shared__ float ss[16][64 + 4];
    const int ch = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * 64;
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int start = a.ch_start[ch], len = a.ch_len[ch];
    const float* S0 = a.ds + ((int64_t)ch * a.H + h) * a.n * a.p;
    const int lrow = tid >> 2, lcol = (tid & 3) * 4;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < a.n; k0 += 16) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int kk = k0 + lcol + i;
            const bool ok = lrow < len && kk < a.n;
            const int64_t tok = start + lrow;
            as[lcol + i][lrow] = ok ? a.q[tok * a.ldq + (int64_t)h * a.n + kk] * a.cum[tok * a.ldc + (int64_t)h * a.n + kk] : 0.f;
        }
        {   // the state tile: thread (k = tid / 16, four neighbouring columns)
            const int sk = k0 + (tid >> 4), sc = c0 + (tid & 15) * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                ss[tid >> 4][(tid & 15) * 4 + i] = (sk < a.n && sc + i < a.p) ? S0[(int64_t)sk * a.p + sc + i] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            float x[4], y[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                x[i] = as[kk][ty * 4 + i];
                y[i] = ss[kk][tx * 4 + i];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(x[i], y[j], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int t = ty * 4 + i;
        if (t >= len) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = c0 + tx * 4 + j;
            if (c < a.p) a.out[(int64_t)(start + t) * a.ldo + (int64_t)h * a.p + c] += acc[i][j];
        }
    }
}

__global__ __launch_bounds__(256) void gate_lower_bound_kernel(float* q, int64_t ldq, float* f, int64_t ldf,
                                                               const float* bias, const float* lower, int T, int n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)T * n) return;
    const int t = (int)(i / n), c = (int)(i % n);
    float* qp = q + (int64_t)t * ldq + c;
    float* fp = f + (int64_t)t * ldf + c;
    *qp = silu_f(*qp);
    const float l = lower[c], z = *fp + (bias ? bias[c] : 0.f);
    *fp = fmaf(1.0f - l, 1.0f / (1.0f + expf(-z)), l);
}

__global__ __launch_bounds__(256) void rotary_pairs_kernel(float* x, int64_t ld, const double* inv_freq,
                                                           const int* tok_pos, int T, int heads, int dim, int rot,
                                                           float scale) {
    const int half = rot / 2, per = dim - half;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)T * heads * per) return;
    const int j = (int)(i % per), hh = (int)((i / per) % heads), t = (int)(i / ((int64_t)per * heads));
    float* p = x + (int64_t)t * ld + (int64_t)hh * dim;
    if (j < half) {
        const double ang = (double)tok_pos[t] * inv_freq[j];
        const float cs = (float)cos(ang), sn = (float)sin(ang);
        const float u = p[j], v = p[j + half];
        p[j] = (u * cs - v * sn) * scale;
        p[j + half] = (v * cs + u * sn) * scale;
    } else {
        p[j + half] *= scale;
    }
}

template <bool F32>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* y, int64_t ldy, const float* gate,
                                                               int64_t ldg, const float* w, void* out_, int64_t ldo,
                                                               int rows, int n, int groups, int gate_first,
                                                               float eps) {
    typedef typename ActS<F32>::T T;
    T* out = (T*)out_;
    const int unit = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (unit >= rows * groups) return;
    const int row = unit / groups, g = unit % groups, gs = n / groups;
    const float* yr = y + (int64_t)row * ldy + (int64_t)g * gs;
    const float* gr = gate + (int64_t)row * ldg + (int64_t)g * gs;
    float ss = 0.f;
    for (int c = lane; c < gs; c += 64) {
        const float u = gate_first ? yr[c] * silu_f(gr[c]) : yr[c];
        ss += u * u;
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
    for (int c = lane; c < gs; c += 64) {
        float u = gate_first ? (yr[c] * silu_f(gr[c])) * inv : (yr[c] * inv) * silu_f(gr[c]);
        if (w) u *= w[g * gs + c];
        ActS<F32>::st(out + (int64_t)row * ldo + (int64_t)g * gs + c, u);
    }
}

struct PagedRows {
    const int* tok_row;
    const int* tok_pos;
    const int* block_table;
    int bt_stride, page;
};

template <bool F32>
__global__ __launch_bounds__(256) void qk_unitnorm_store_kernel(float* qkv, int64_t ld, void* kc_, void* vc_,
                                                                PagedRows pr, int T, int H, int G, int d, int dv,
                                                                float eps) {
    typedef typename ActS<F32>::T T_;
    T_* kc = (T_*)kc_;
    T_* vc = (T_*)vc_;
    const int per = H + 2 * G;
    const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (unit >= (int64_t)T * per) return;
    const int t = (int)(unit / per), u = (int)(unit % per);
    float* row = qkv + (int64_t)t * ld;
    const int pos = pr.tok_pos[t];
    const int pg = pr.block_table[(int64_t)pr.tok_row[t] * pr.bt_stride + pos / pr.page];
    const int64_t slot = (int64_t)pg * pr.page + pos % pr.page;
    if (u < H + G) {
        float* p = row + (u < H ? (int64_t)u * d : (int64_t)H * d + (int64_t)(u - H) * d);
        float ss = 0.f;
        for (int c = lane; c < d; c += 64) ss += p[c] * p[c];
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)d + eps);
        if (u < H) {
            for (int c = lane; c < d; c += 64) p[c] = p[c] * inv;
        } else if (pg >= 0) {
            T_* dst = kc + (slot * G + (u - H)) * d;
            for (int c = lane; c < d; c += 64) ActS<F32>::st(dst + c, p[c] * inv);
        }
    } else if (pg >= 0) {
        const int g = u - H - G;
        const float* p = row + (int64_t)(H + G) * d + (int64_t)g * dv;
        T_* dst = vc + (slot * G + g) * dv;
        for (int c = lane; c < dv; c += 64) ActS<F32>::st(dst + c, p[c]);
    }
}

// One wave per (token, `hpw` consecutive query or key heads: the sines and cosines of a position are formed once for
// them).  q [T, ld]: heads * d query values then kv_heads * d key values, as one projection leaves them.  The query gets its bias and rotation in place; the key goes, with its bias, unrotated
// into the value page and rotated into the key page.  angle = position * inv_freq[i], formed in fp64.
template <bool F32>
__global__ __launch_bounds__(256) void qk_rotary_store_kernel(float* qk, int64_t ld, const float* qb, const float* kb,
                                                              void* kc_, void* vc_, const double* inv_freq,
                                                              PagedRows pr, int T, int H, int G, int d, int rot,
                                                              int adjacent, int hpw, unsigned rot_blocks, const float* act_in,
                                                              int64_t lda, void* act_out, int64_t ldao, int act_n,
                                                              int act_kind, float act_limit, float act_slope) {
    typedef typename ActS<F32>::T T_;
    if (blockIdx.x >= rot_blocks) {
        // the workgroups behind the rotation's: the gate of a feed-forward whose gate | up columns came out of the
        // same projection (a parallel layer), so that the step needs no launch of its own
        const unsigned b = blockIdx.x - rot_blocks, cb = (act_n + 255) / 256;
        const int64_t row = b / cb;
        const int c = (b % cb) * 256 + threadIdx.x;
        if (c < act_n)
            ActS<F32>::st((T_*)act_out + row * ldao + c,
                          gated_act_f(act_in[row * lda + c], act_in[row * lda + act_n + c], act_kind, act_limit, act_slope));
        return;
    }
    T_* kc = (T_*)kc_;
    T_* vc = (T_*)vc_;
    const int per = H + G, groups = (per + hpw - 1) / hpw;
    const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (unit >= (int64_t)T * groups) return;
    const int t = (int)(unit / groups), u0 = (int)(unit % groups) * hpw, u1 = u0 + hpw < per ? u0 + hpw : per;
    const int pos = pr.tok_pos[t];
    float* row = qk + (int64_t)t * ld;
    int64_t slot = -1;            // the token's place in the pages (needed where the wave holds a key head)
    if (u1 > H) {
        const int pg = pr.block_table[(int64_t)pr.tok_row[t] * pr.bt_stride + pos / pr.page];
        if (pg >= 0) slot = ((int64_t)pg * pr.page + pos % pr.page) * G;
    }
    const int half = rot / 2;
    for (int i = lane; i < half; i += 64) {
        const int a = adjacent ? 2 * i : i, b = adjacent ? 2 * i + 1 : i + half;
        const double ang = (double)pos * inv_freq[i];
        const float cs = (float)cos(ang), sn = (float)sin(ang);     // once for all heads of the wave
        for (int u = u0; u < u1; ++u) {
            float* p = row + (int64_t)u * d;
            const float* bias = u < H ? (qb ? qb + (int64_t)u * d : nullptr) : (kb ? kb + (int64_t)(u - H) * d : nullptr);
            const float x0 = bias ? p[a] + bias[a] : p[a], x1 = bias ? p[b] + bias[b] : p[b];
            const float r0 = x0 * cs - x1 * sn, r1 = x1 * cs + x0 * sn;
            if (u < H) {
                p[a] = r0;
                p[b] = r1;
            } else if (slot >= 0) {
                T_* kdst = kc + (slot + (u - H)) * d;
                T_* vdst = vc + (slot + (u - H)) * d;
                ActS<F32>::st(kdst + a, r0);
                ActS<F32>::st(kdst + b, r1);
                ActS<F32>::st(vdst + a, x0);
                ActS<F32>::st(vdst + b, x1);
            }
        }
    }
    for (int u = u0; u < u1; ++u) {
        float* p = row + (int64_t)u * d;
        const float* bias = u < H ? (qb ? qb + (int64_t)u * d : nullptr) : (kb ? kb + (int64_t)(u - H) * d : nullptr);
        for (int c = rot + lane; c < d; c += 64) {
            const float x0 = bias ? p[c] + bias[c] : p[c];
            if (u < H) {
                p[c] = x0;
            } else if (slot >= 0) {
                ActS<F32>::st(kc + (slot + (u - H)) * d + c, x0);
                ActS<F32>::st(vc + (slot + (u - H)) * d + c, x0);
            }
        }
    }
}

// value of channel c at token t under a causal convolution of `taps` taps whose first inputs come from the slot
__device__ __forceinline__ float conv_at(const float* in, int64_t ldi, const float* state, const float* w,
                                         const StepRows& r, int t, int c, int C, int taps) {
    const int b = r.tok_row[t];
    const int rel = t - r.row_start[b];
    const bool carried = r.row_ctx[b] > 0;
    const float* st = state + ((int64_t)r.row_slot[b] * (taps - 1)) * C + c;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int src = rel - (taps - 1) + j;
        float v;
        if (src >= 0) v = in[(int64_t)(t - (taps - 1) + j) * ldi + c];
        else v = carried ? st[(int64_t)(src + taps - 1) * C] : 0.f;
        acc = fmaf(w[(int64_t)c * taps + j], v, acc);
    }
    return acc;
}

template <bool F32>
__global__ __launch_bounds__(256) void conv_taps_kernel(const float* in, int64_t ldi, const float* state,
                                                        const float* w, float* o32, int64_t ld32, void* oact_,
                                                        int64_t ldoa, int add_input, StepRows r, int T, int C,
                                                        int taps) {
    typedef typename ActS<F32>::T T_;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)T * C) return;
    const int t = (int)(i / C), c = (int)(i % C);
    float v = conv_at(in, ldi, state, w, r, t, c, C, taps);
    if (add_input) v += in[(int64_t)t * ldi + c];
    if (o32) o32[(int64_t)t * ld32 + c] = v;
    if (oact_) ActS<F32>::st((T_*)oact_ + (int64_t)t * ldoa + c, v);
}

// columns [0, Cq) -> q (fp32), [Cq, Cq + Ck) -> the token's row of the key page, the last Cv -> the value page.
// w == NULL: no convolution, the columns go where they belong as they are
template <bool F32>
__global__ __launch_bounds__(256) void conv_qkv_store_kernel(const float* in, int64_t ldi, const float* state,
                                                             const float* w, float* q, int64_t ldq, void* kc_,
                                                             void* vc_, StepRows r, PagedRows pr, int T, int Cq,
                                                             int Ck, int Cv, int taps) {
    typedef typename ActS<F32>::T T_;
    const int C = Cq + Ck + Cv;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)T * C) return;
    const int t = (int)(i / C), c = (int)(i % C);
    const float v = w ? conv_at(in, ldi, state, w, r, t, c, C, taps) : in[(int64_t)t * ldi + c];
    if (c < Cq) {
        q[(int64_t)t * ldq + c] = v;
        return;
    }
    const int pos = pr.tok_pos[t];
    const int pg = pr.block_table[(int64_t)pr.tok_row[t] * pr.bt_stride + pos / pr.page];
    if (pg < 0) return;
    const int64_t slot = (int64_t)pg * pr.page + pos % pr.page;
    if (c < Cq + Ck) ActS<F32>::st((T_*)kc_ + slot * Ck + (c - Cq), v);
    else ActS<F32>::st((T_*)vc_ + slot * Cv + (c - Cq - Ck), v);
}

constexpr int kMaxVC = 4;  // value columns per lane: vdim <= 256

// One workgroup per (token, head).  Its NW waves (4, or 16 when a step has too few tokens to fill the
// chip otherwise: decoding) take the window's 64-key tiles in turn: a lane scores
// one key (q from LDS, the key row straight from its page), the wave forms max / sum of the tile and
// then, lanes now owning value columns, adds the tile's weighted values; the waves' partial softmaxes
// meet in LDS.  The same code serves a prompt's portion and a single decoded token.  Positions below
// `keep_first` stay visible after the window has passed them (a second run of tiles, at their true
// positions); sinks[h] joins the denominator as exp(sink) with no key and no value.
template <bool F32, int NW>
__global__ __launch_bounds__(64 * NW) void window_attn_kernel(const float* q, int64_t ldq, const void* kc_,
                                                          const void* vc_, void* out_, int64_t ldo, PagedRows pr,
                                                          const float* slopes, int T, int H, int G, int d, int dv,
                                                          float scale, int window, const int* row_len, int max_len,
                                                          int keep_first, const float* sinks) {
    typedef typename ActS<F32>::T T_;
    extern __shared__ float lds[];
    if (max_len > 0 && row_len[pr.tok_row[blockIdx.x / H]] > max_len) return;   // the tiled kernel's rows
    const T_* kc = (const T_*)kc_;
    const T_* vc = (const T_*)vc_;
    T_* out = (T_*)out_;
    const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float* qs = lds;
    float* ps = lds + d + wv * 64;
    float* mm = lds + d + 64 * NW;
    float* ll = mm + NW;
    float* aa = ll + NW;
    const int t = blockIdx.x / H, h = blockIdx.x % H, g = h / (H / G);
    const int pos = pr.tok_pos[t];
    const int* bt = pr.block_table + (int64_t)pr.tok_row[t] * pr.bt_stride;
    const int lo = pos - window + 1 > 0 ? pos - window + 1 : 0;
    const float slope = slopes ? slopes[h] : 0.f;
    for (int c = threadIdx.x; c < d; c += 64 * NW) qs[c] = q[(int64_t)t * ldq + (int64_t)h * d + c];
    __syncthreads();
    float m = -INFINITY, l = 0.f, acc[kMaxVC] = {0.f, 0.f, 0.f, 0.f};
    const int kept = keep_first < lo ? keep_first : lo;    // kept positions the window no longer covers: [0, kept)
    for (int run = kept > 0 ? 0 : 1; run < 2; ++run) {
    const int first = run ? lo : 0, last = run ? pos : kept - 1;
    for (int j0 = first + 64 * wv; j0 <= last; j0 += 64 * NW) {
        const int j = j0 + lane;
        float s = -INFINITY;
        if (j <= last) {
            const int pg = bt[j / pr.page];
            const T_* kr = kc + (((int64_t)pg * pr.page + j % pr.page) * G + g) * d;
            float dot = 0.f;
            if (!F32 && (d & 7) == 0) {
                for (int c = 0; c < d; c += 8) {
                    const uint4 kv = ld16(kr + c);
                    const uint32_t w[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        dot = fmaf(qs[c + 2 * e], bf16_lo(w[e]), dot);
                        dot = fmaf(qs[c + 2 * e + 1], bf16_hi(w[e]), dot);
                    }
                }
            } else {
                for (int c = 0; c < d; ++c) dot = fmaf(qs[c], ActS<F32>::ld(kr + c), dot);
            }
            s = dot * scale - slope * (float)(pos - j);
        }
        const float mn = fmaxf(m, wave_max(s));
        const float pj_ = j <= last ? expf(s - mn) : 0.f;
        const float corr = expf(m - mn);   // m = -inf on the wave's first tile: exp(-inf) = 0
        l = l * corr + wave_sum(pj_);
        m = mn;
        __builtin_amdgcn_wave_barrier();
        ps[lane] = pj_;
        __builtin_amdgcn_wave_barrier();
        const int cnt = last - j0 + 1 < 64 ? last - j0 + 1 : 64;
#pragma unroll
        for (int ci = 0; ci < kMaxVC; ++ci) acc[ci] *= corr;
        // eight value rows at a time, their loads in flight together (a tile of 64 keys lies in two pages at
        // most when a page holds 64 tokens or more: their ids are looked up once)
        const int pA = j0 / pr.page;
        const bool two = pr.page >= 64;
        const int pgA = bt[pA], pgB = (two && (j0 + cnt - 1) / pr.page != pA) ? bt[pA + 1] : pgA;
        for (int jj = 0; jj < cnt; jj += 8) {
            float pj[8];
            const T_* vr[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const bool ok = jj + u < cnt;
                const int jk = ok ? j0 + jj + u : j0;
                const int pg = two ? (jk / pr.page == pA ? pgA : pgB) : bt[jk / pr.page];
                vr[u] = vc + (((int64_t)pg * pr.page + jk % pr.page) * G + g) * dv;
                pj[u] = ok ? ps[jj + u] : 0.f;
            }
#pragma unroll
            for (int ci = 0; ci < kMaxVC; ++ci) {
                const int c = lane + ci * 64;
                if (c < dv) {
                    float x[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) x[u] = ActS<F32>::ld(vr[u] + c);
#pragma unroll
                    for (int u = 0; u < 8; ++u) acc[ci] = fmaf(pj[u], x[u], acc[ci]);
                }
            }
        }
    }
    }
    if (lane == 0) {
        mm[wv] = m;
        ll[wv] = l;
    }
#pragma unroll
    for (int ci = 0; ci < kMaxVC; ++ci) {
        const int c = lane + ci * 64;
        if (c < dv) aa[wv * dv + c] = acc[ci];
    }
    __syncthreads();
    if (wv == 0) {
        float M = mm[0];                                   // wave 0 always has a key: finite
#pragma unroll
        for (int w = 1; w < NW; ++w) M = fmaxf(M, mm[w]);
        float L = 0.f;
        if (sinks) {
            M = fmaxf(M, sinks[h]);
            L = expf(sinks[h] - M);
        }
        float w4[NW];
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            w4[w] = expf(mm[w] - M);   // a wave without keys: exp(-inf) = 0
            L = fmaf(ll[w], w4[w], L);
        }
#pragma unroll
        for (int ci = 0; ci < kMaxVC; ++ci) {
            const int c = lane + ci * 64;
            if (c < dv) {
                float o = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) o = fmaf(aa[w * dv + c], w4[w], o);
                ActS<F32>::st(out + (int64_t)t * ldo + (int64_t)h * dv + c, o / L);
            }
        }
    }
}


// The same attention for steps of few tokens (decoding), where one workgroup per (token, head) leaves most of the chip
// idle and every query head of a key/value head reads the same pages again: one workgroup of four waves per (token,
// key/value head, group of up to eight of its query heads, split of the key tiles).  A wave takes 64-key tiles - those
// of the kept first positions, then the window's - in steps of 4 * splits; a lane scores ONE key for all heads of the
// group from one read of it, the heads' softmax pieces go through LDS, and the weighted values are gathered with
// 16-byte loads (dv / VEC lanes per value row, several rows per load; `vec` == 0: a lane per value column).  The
// waves' partial softmaxes meet in LDS; with splits > 1 the workgroup leaves (max, sum, weighted values) in `part`
// for window_attn_merge_kernel, which also adds the sink.
constexpr int kGrpMax = 8;

template <bool F32, int RT>
__global__ __launch_bounds__(256) void window_attn_group_kernel(const float* q, int64_t ldq, const void* kc_,
                                                                const void* vc_, void* out_, int64_t ldo, float* part,
                                                                PagedRows pr, const float* slopes, const float* sinks,
                                                                int H, int G, int d, int dv, float scale, int window,
                                                                int keep_first, const int* row_len, int max_len,
                                                                int splits, int vec) {
    typedef typename ActS<F32>::T T_;
    constexpr int VEC = F32 ? 4 : 8;
    extern __shared__ float lds[];
    const T_* kc = (const T_*)kc_;
    const T_* vc = (const T_*)vc_;
    const int R = H / G, ngrp = (R + kGrpMax - 1) / kGrpMax;
    const int unit = blockIdx.x, split = blockIdx.y;
    const int t = unit / (G * ngrp), g = (unit / ngrp) % G, grp = unit % ngrp;
    if (max_len > 0 && row_len[pr.tok_row[t]] > max_len) return;   // the tiled kernel's rows
    const int h0 = g * R + grp * kGrpMax;
    const int nh = R - grp * kGrpMax < kGrpMax ? R - grp * kGrpMax : kGrpMax;   // heads of this workgroup, <= RT
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
    float* qs = lds;                    // [RT][d]
    float* ps = qs + RT * d;            // [4][RT][64]
    float* red = ps + 4 * RT * 64;      // [4][RT][dv]
    float* mm = red + 4 * RT * dv;      // [4][RT]
    float* ll = mm + 4 * RT;            // [4][RT]
    for (int i = tid; i < RT * d; i += 256) {
        const int r = i / d;
        qs[i] = r < nh ? q[(int64_t)t * ldq + (int64_t)(h0 + r) * d + (i - r * d)] : 0.f;
    }
    __syncthreads();
    const int pos = pr.tok_pos[t];
    const int* bt = pr.block_table + (int64_t)pr.tok_row[t] * pr.bt_stride;
    const int lo = pos - window + 1 > 0 ? pos - window + 1 : 0;
    const int kept = keep_first < lo ? keep_first : lo;
    const int nk = (kept + 63) / 64, nw = (pos - lo) / 64 + 1;
    float m[RT], l[RT], slope[RT], acc[RT][8];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        m[r] = -INFINITY;
        l[r] = 0.f;
        slope[r] = (slopes && r < nh) ? slopes[h0 + r] : 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[r][e] = 0.f;
    }
    const int lpr = vec ? dv / VEC : 1, rp = vec ? 64 / lpr : 1;   // lanes per value row, rows per load
    const int sub = lane / lpr, cb = lane - sub * lpr;
    float* pw = ps + wv * RT * 64;
    for (int u = split * 4 + wv; u < nk + nw; u += 4 * splits) {
        const int first = u < nk ? 64 * u : lo + 64 * (u - nk);
        const int end = u < nk ? kept - 1 : pos;
        const int last = first + 63 < end ? first + 63 : end;
        const int j = first + lane;
        const bool valid = j <= last;
        float dot[RT];
#pragma unroll
        for (int r = 0; r < RT; ++r) dot[r] = 0.f;
        if (valid) {
            const T_* kr = kc + (((int64_t)bt[j / pr.page] * pr.page + j % pr.page) * G + g) * d;
            if (!F32 && (d & 7) == 0) {
                // four 16-byte pieces of the key row in flight at a time
                for (int c0 = 0; c0 < d; c0 += 32) {
                    uint4 kq[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) kq[u] = c0 + 8 * u < d ? ld16(kr + c0 + 8 * u) : make_uint4(0, 0, 0, 0);
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int c = c0 + 8 * u;
                        if (c >= d) break;
                        const uint4 kv = kq[u];
                        const float k8[8] = {bf16_lo(kv.x), bf16_hi(kv.x), bf16_lo(kv.y), bf16_hi(kv.y),
                                             bf16_lo(kv.z), bf16_hi(kv.z), bf16_lo(kv.w), bf16_hi(kv.w)};
#pragma unroll
                        for (int r = 0; r < RT; ++r) {
                            const float4 qa = *reinterpret_cast<const float4*>(qs + r * d + c);
                            const float4 qb = *reinterpret_cast<const float4*>(qs + r * d + c + 4);
                            dot[r] = fmaf(qa.x, k8[0], dot[r]);
                            dot[r] = fmaf(qa.y, k8[1], dot[r]);
                            dot[r] = fmaf(qa.z, k8[2], dot[r]);
                            dot[r] = fmaf(qa.w, k8[3], dot[r]);
                            dot[r] = fmaf(qb.x, k8[4], dot[r]);
                            dot[r] = fmaf(qb.y, k8[5], dot[r]);
                            dot[r] = fmaf(qb.z, k8[6], dot[r]);
                            dot[r] = fmaf(qb.w, k8[7], dot[r]);
                        }
                    }
                }
            } else {
                for (int c = 0; c < d; ++c) {
                    const float kf = ActS<F32>::ld(kr + c);
#pragma unroll
                    for (int r = 0; r < RT; ++r) dot[r] = fmaf(qs[r * d + c], kf, dot[r]);
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const float sc = valid ? dot[r] * scale - slope[r] * (float)(pos - j) : -INFINITY;
            const float mn = fmaxf(m[r], wave_max(sc));        // finite: a tile holds at least one key
            const float pj = valid ? expf(sc - mn) : 0.f;
            const float corr = expf(m[r] - mn);                // m = -inf on the wave's first tile: exp(-inf) = 0
            l[r] = l[r] * corr + wave_sum(pj);
            m[r] = mn;
            pw[r * 64 + lane] = pj;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[r][e] *= corr;
        }
        __builtin_amdgcn_wave_barrier();
        const int cnt = last - first + 1;
        if (vec) {
            if (sub < rp) {
                // a tile of 64 keys lies in two pages at most when a page holds 64 tokens or more: their ids are looked
                // up once; eight value rows in flight at a time
                const int pA = first / pr.page;
                const bool two = pr.page >= 64;
                const int pgA = bt[pA], pgB = (two && last / pr.page != pA) ? bt[pA + 1] : pgA;
                for (int row0 = sub; row0 < cnt; row0 += 8 * rp) {
                    uint4 vq[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int row = row0 + u * rp;
                        const int jk = first + (row < cnt ? row : 0);
                        const int pg = two ? (jk / pr.page == pA ? pgA : pgB) : bt[jk / pr.page];
                        vq[u] = ld16(vc + (((int64_t)pg * pr.page + jk % pr.page) * G + g) * dv + cb * VEC);
                    }
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int row = row0 + u * rp;
                        if (row >= cnt) break;
                        const uint4 vv = vq[u];
                        float v8[8];
                        if (F32) {
                            v8[0] = __uint_as_float(vv.x); v8[1] = __uint_as_float(vv.y);
                            v8[2] = __uint_as_float(vv.z); v8[3] = __uint_as_float(vv.w);
                            v8[4] = v8[5] = v8[6] = v8[7] = 0.f;
                        } else {
                            v8[0] = bf16_lo(vv.x); v8[1] = bf16_hi(vv.x); v8[2] = bf16_lo(vv.y); v8[3] = bf16_hi(vv.y);
                            v8[4] = bf16_lo(vv.z); v8[5] = bf16_hi(vv.z); v8[6] = bf16_lo(vv.w); v8[7] = bf16_hi(vv.w);
                        }
#pragma unroll
                        for (int r = 0; r < RT; ++r) {
                            const float w = pw[r * 64 + row];
#pragma unroll
                            for (int e = 0; e < VEC; ++e) acc[r][e] = fmaf(w, v8[e], acc[r][e]);
                        }
                    }
                }
            }
        } else {
            for (int row = 0; row < cnt; ++row) {
                const int jk = first + row;
                const T_* vr = vc + (((int64_t)bt[jk / pr.page] * pr.page + jk % pr.page) * G + g) * dv;
#pragma unroll
                for (int ci = 0; ci < kMaxVC; ++ci) {
                    const int c = lane + ci * 64;
                    if (c < dv) {
                        const float x = ActS<F32>::ld(vr + c);
#pragma unroll
                        for (int r = 0; r < RT; ++r) acc[r][ci] = fmaf(pw[r * 64 + row], x, acc[r][ci]);
                    }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            mm[wv * RT + r] = m[r];
            ll[wv * RT + r] = l[r];
        }
    }
    float* rw = red + wv * RT * dv;
    if (vec) {
        // the row groups of a wave add their sums one after the other
        for (int s2 = 0; s2 < rp; ++s2) {
            if (sub == s2) {
#pragma unroll
                for (int r = 0; r < RT; ++r)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const int i = r * dv + cb * VEC + e;
                        rw[i] = (s2 == 0 ? 0.f : rw[i]) + acc[r][e];
                    }
            }
            __builtin_amdgcn_wave_barrier();
        }
    } else {
#pragma unroll
        for (int ci = 0; ci < kMaxVC; ++ci) {
            const int c = lane + ci * 64;
            if (c < dv)
#pragma unroll
                for (int r = 0; r < RT; ++r) rw[r * dv + c] = acc[r][ci];
        }
    }
    __syncthreads();
    for (int i = tid; i < nh * dv; i += 256) {
        const int r = i / dv, c = i - r * dv;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) M = fmaxf(M, mm[w * RT + r]);
        float L = 0.f, o = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float mw = mm[w * RT + r];
            const float f = mw == -INFINITY ? 0.f : expf(mw - M);     // a wave (or a whole split) without keys
            L = fmaf(ll[w * RT + r], f, L);
            o = fmaf(red[(w * RT + r) * dv + c], f, o);
        }
        const int h = h0 + r;
        if (splits == 1) {
            if (sinks) {
                const float sk = sinks[h], mf = fmaxf(M, sk), f = expf(M - mf);
                L = L * f + expf(sk - mf);
                o *= f;
            }
            ActS<F32>::st((T_*)out_ + (int64_t)t * ldo + (int64_t)h * dv + c, o / L);
        } else {
            float* dst = part + (((int64_t)t * H + h) * splits + split) * (dv + 2);
            if (c == 0) {
                dst[0] = M;
                dst[1] = L;
            }
            dst[2 + c] = o;
        }
    }
}

// one wave per (token, head): the splits' pieces and the sink become the output row
template <bool F32>
__global__ __launch_bounds__(64) void window_attn_merge_kernel(const float* part, void* out_, int64_t ldo,
                                                               const int* tok_row, const float* sinks, int H, int dv,
                                                               int splits, const int* row_len, int max_len) {
    typedef typename ActS<F32>::T T_;
    const int t = blockIdx.x / H, h = blockIdx.x % H, lane = threadIdx.x;
    if (max_len > 0 && row_len[tok_row[t]] > max_len) return;
    const float* src = part + (int64_t)blockIdx.x * splits * (dv + 2);
    float M = sinks ? sinks[h] : -INFINITY;
    for (int s2 = 0; s2 < splits; ++s2) M = fmaxf(M, src[(int64_t)s2 * (dv + 2)]);
    float L = sinks ? expf(sinks[h] - M) : 0.f;
    for (int s2 = 0; s2 < splits; ++s2) {
        const float ms = src[(int64_t)s2 * (dv + 2)];
        if (ms != -INFINITY) L = fmaf(src[(int64_t)s2 * (dv + 2) + 1], expf(ms - M), L);
    }
    for (int c = lane; c < dv; c += 64) {
        float o = 0.f;
        for (int s2 = 0; s2 < splits; ++s2) {
            const float ms = src[(int64_t)s2 * (dv + 2)];
            if (ms != -INFINITY) o = fmaf(src[(int64_t)s2 * (dv + 2) + 2 + c], expf(ms - M), o);
        }
        ActS<F32>::st((T_*)out_ + (int64_t)t * ldo + (int64_t)h * dv + c, o / L);
    }
}

// The same attention for a prompt's portion, bf16 keys and values: one workgroup per (64 consecutive tokens
// of a row, head).  Key tiles are pages (64 tokens) staged once in LDS for all 64 queries; q.k on
// v_mfma_f32_16x16x32_bf16 (q rounded to bf16 as the keys are), scores, distance penalty, mask and softmax
// in fp32 per lane, and P.V with every fp32 weight split exactly into three bf16 numbers, on the same bf16
// instruction with fp32 accumulators: the score accumulators of a lane, S[key 16 nt + 4 (lane / 16) + j][query
// lane % 16], serve as its second operand where they lie, so P never leaves the registers.
typedef __attribute__((ext_vector_type(8))) __bf16 wa_bf16x8_t;

template <int KS, int CT>
__global__ __launch_bounds__(256) void window_attn_tile_kernel(const float* q, int64_t ldq, const uint16_t* kc,
                                                               const uint16_t* vc, uint16_t* out, int64_t ldo,
                                                               PagedRows pr, const int* ch_start, const int* ch_len,
                                                               const float* slopes, int H, int G, float scale,
                                                               int window, int keep_first, const float* sinks) {
    constexpr int D = KS * 32, DV = CT * 16, SK = D + 8, SV = DV + 8;
    __shared__ __attribute__((aligned(16))) uint16_t Ks[64][SK];
    // values as pairs of neighbouring keys: dword [i][c] = V[2i][c] | V[2i+1][c] << 16, which is how the matrix
    // instruction wants them (two contraction slots per register)
    __shared__ __attribute__((aligned(16))) uint32_t Vp[32][SV];
    const int ch = blockIdx.x, h = blockIdx.y, g = h / (H / G);
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, r = lane & 15, qd = lane >> 4;
    const int start = ch_start[ch], len = ch_len[ch];
    const int* bt = pr.block_table + (int64_t)pr.tok_row[start] * pr.bt_stride;
    const int p0 = pr.tok_pos[start];            // positions run on from here within the chunk
    const int myq = 16 * wv + r;
    const bool qok = myq < len;
    const int qpos = p0 + myq;
    wa_bf16x8_t qf[KS];
    {
        const float* qp = q + (int64_t)(start + (qok ? myq : 0)) * ldq + (int64_t)h * D + 8 * qd;
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            const float4 a = *reinterpret_cast<const float4*>(qp + 32 * kk);
            const float4 b = *reinterpret_cast<const float4*>(qp + 32 * kk + 4);
            const uint4 pk = make_uint4(pack_bf16x2(a.x, a.y), pack_bf16x2(a.z, a.w), pack_bf16x2(b.x, b.y),
                                        pack_bf16x2(b.z, b.w));
            qf[kk] = __builtin_bit_cast(wa_bf16x8_t, pk);
        }
    }
    float m = -INFINITY, l = 0.f;
    f32x4_t o[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) o[ct] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const float slope = slopes ? slopes[h] : 0.f;
    const int klo = p0 - window + 1 > 0 ? p0 - window + 1 : 0, khi = p0 + len - 1;
    const int wq_lo = p0 + 16 * wv, wq_hi = wq_lo + 15;   // this wave's query positions
    // key tiles: those of the kept first positions that the window of the chunk's first query has left behind,
    // then the window's
    const int kt_lo = klo / 64, kt_keep = ((keep_first < klo ? keep_first : klo) + 63) / 64;
    for (int kt = kt_keep > 0 ? 0 : kt_lo; kt <= khi / 64; kt = (kt + 1 >= kt_keep && kt + 1 < kt_lo) ? kt_lo : kt + 1) {
        const int kbase = kt * 64;
        const int64_t pgrow = (int64_t)bt[kt] * 64;
        __syncthreads();
        for (int i = tid; i < 64 * (D / 8); i += 256) {
            const int rr = i / (D / 8), cc = i % (D / 8);
            st16(&Ks[rr][cc * 8], ld16(kc + ((pgrow + rr) * G + g) * D + cc * 8));
        }
        for (int i = tid; i < 32 * (DV / 8); i += 256) {
            const int rr = i / (DV / 8), cc = i % (DV / 8);
            const uint4 a = ld16(vc + ((pgrow + 2 * rr) * G + g) * DV + cc * 8);
            const uint4 b = ld16(vc + ((pgrow + 2 * rr + 1) * G + g) * DV + cc * 8);
            st16(&Vp[rr][cc * 8], make_uint4((a.x & 0xffffu) | (b.x << 16), (a.x >> 16) | (b.x & 0xffff0000u),
                                             (a.y & 0xffffu) | (b.y << 16), (a.y >> 16) | (b.y & 0xffff0000u)));
            st16(&Vp[rr][cc * 8 + 4], make_uint4((a.z & 0xffffu) | (b.z << 16), (a.z >> 16) | (b.z & 0xffff0000u),
                                                 (a.w & 0xffffu) | (b.w << 16), (a.w >> 16) | (b.w & 0xffff0000u)));
        }
        __syncthreads();
        // nothing of this tile is visible to the wave
        if (kbase > wq_hi || (kbase + 63 <= wq_lo - window && kbase >= keep_first)) continue;
        f32x4_t sc[4];
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
            sc[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) {
                const wa_bf16x8_t kf = __builtin_bit_cast(wa_bf16x8_t, ld16(&Ks[16 * nt + r][32 * kk + 8 * qd]));
                sc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[kk], sc[nt], 0, 0, 0);
            }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int kpos = kbase + 16 * nt + 4 * qd + j;
                const bool ok = qok && kpos <= qpos && (kpos > qpos - window || kpos < keep_first);
                const float v = ok ? sc[nt][j] * scale - slope * (float)(qpos - kpos) : -INFINITY;
                sc[nt][j] = v;
                mx = fmaxf(mx, v);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mn = fmaxf(m, mx);
        constexpr float kLog2e = 1.4426950408889634f;      // e^x as 2^(x log2 e) on the hardware's exp2
        const float corr = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m - mn) * kLog2e);
        float ps = 0.f;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float pv = sc[nt][j] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((sc[nt][j] - mn) * kLog2e);
                sc[nt][j] = pv;
                ps += pv;
            }
        ps += __shfl_xor(ps, 16, 64);
        ps += __shfl_xor(ps, 32, 64);
        l = l * corr + ps;
        m = mn;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) o[ct] *= corr;
        // P.V with P kept whole: an fp32 weight is the exact sum of three bf16 numbers (its leading 8, the next 8
        // and the last 8 bits of the mantissa, each cut off, not rounded), the values are bf16 as cached, so three
        // bf16 matrix instructions with fp32 accumulators form the same products as one in fp32 would - at three
        // eighths of its cost.  The contraction index of the instruction is only a label: slot (qd, e) of both
        // operands stands for key 32 kb + 16 (e / 4) + 4 qd + e % 4, which is where the lane's scores already lie.
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            uint32_t hi[4], mid[4], lo[4];
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {       // two weights per dword
                uint32_t h2[2], m2[2], l2[2];
#pragma unroll
                for (int x = 0; x < 2; ++x) {
                    const int e = 2 * e2 + x;
                    const float pv = sc[2 * kb + e / 4][e % 4];
                    const uint32_t hb = __float_as_uint(pv) & 0xffff0000u;
                    const float r1 = pv - __uint_as_float(hb);
                    const uint32_t mb = __float_as_uint(r1) & 0xffff0000u;
                    const float r2 = r1 - __uint_as_float(mb);
                    h2[x] = hb;
                    m2[x] = mb;
                    l2[x] = __float_as_uint(r2) & 0xffff0000u;
                }
                hi[e2] = (h2[0] >> 16) | h2[1];
                mid[e2] = (m2[0] >> 16) | m2[1];
                lo[e2] = (l2[0] >> 16) | l2[1];
            }
            const wa_bf16x8_t ph = __builtin_bit_cast(wa_bf16x8_t, make_uint4(hi[0], hi[1], hi[2], hi[3]));
            const wa_bf16x8_t pm = __builtin_bit_cast(wa_bf16x8_t, make_uint4(mid[0], mid[1], mid[2], mid[3]));
            const wa_bf16x8_t pl = __builtin_bit_cast(wa_bf16x8_t, make_uint4(lo[0], lo[1], lo[2], lo[3]));
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                uint32_t vw[4];
#pragma unroll
                for (int e2 = 0; e2 < 4; ++e2)     // keys k0, k0 + 1 with k0 = 32 kb + 16 (e2 / 2) + 4 qd + 2 (e2 % 2)
                    vw[e2] = Vp[16 * kb + 8 * (e2 / 2) + 2 * qd + (e2 % 2)][16 * ct + r];
                const wa_bf16x8_t vf = __builtin_bit_cast(wa_bf16x8_t, make_uint4(vw[0], vw[1], vw[2], vw[3]));
                o[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, ph, o[ct], 0, 0, 0);
                o[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pm, o[ct], 0, 0, 0);
                o[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pl, o[ct], 0, 0, 0);
            }
        }
    }
    if (qok) {
        float inv = 1.0f / l;
        if (sinks) {   // one more term of the denominator, without a value (m is finite: a query sees itself)
            const float sk = sinks[h], mn = fmaxf(m, sk);
            inv = expf(m - mn) / (l * expf(m - mn) + expf(sk - mn));
        }
        uint16_t* op = out + (int64_t)(start + myq) * ldo + (int64_t)h * DV + 4 * qd;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            uint2 w;
            w.x = pack_bf16x2(o[ct][0] * inv, o[ct][1] * inv);
            w.y = pack_bf16x2(o[ct][2] * inv, o[ct][3] * inv);
            *reinterpret_cast<uint2*>(op + 16 * ct) = w;
        }
    }
}

// groups of a thousand values and more: one workgroup per (row, group)
template <bool F32>
__global__ __launch_bounds__(256) void gated_group_norm_wide_kernel(const float* y, int64_t ldy, const float* gate,
                                                                    int64_t ldg, const float* w, void* out_,
                                                                    int64_t ldo, int n, int groups, int gate_first,
                                                                    float eps) {
    typedef typename ActS<F32>::T T;
    __shared__ float red[4];
    T* out = (T*)out_;
    const int row = blockIdx.x / groups, g = blockIdx.x % groups, gs = n / groups;
    const float* yr = y + (int64_t)row * ldy + (int64_t)g * gs;
    const float* gr = gate + (int64_t)row * ldg + (int64_t)g * gs;
    float ss = 0.f;
    for (int c = threadIdx.x; c < gs; c += 256) {
        const float u = gate_first ? yr[c] * silu_f(gr[c]) : yr[c];
        ss += u * u;
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
    for (int c = threadIdx.x; c < gs; c += 256) {
        float u = gate_first ? (yr[c] * silu_f(gr[c])) * inv : (yr[c] * inv) * silu_f(gr[c]);
        if (w) u *= w[g * gs + c];
        ActS<F32>::st(out + (int64_t)row * ldo + (int64_t)g * gs + c, u);
    }
}

}  // namespace mv

extern "C" {

using mv::StepRows;

int mv_conv_silu(const float* in, int64_t ldi, float* state, const float* w, const float* bias, float* out,
                 int64_t ldo, const int32_t* tok_row, const int32_t* row_start, const int32_t* row_len,
                 const int32_t* row_ctx, const int32_t* row_slot, int tokens, int rows, int channels, int taps,
                 mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || rows < 0 || channels <= 0 || taps < 1 || taps > kMaxTaps) return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!in || (!state && taps > 1) || !w || !out || ldi < channels || ldo < channels) return MV_ERR_INVALID_ARG;
    StepRows r{tok_row, nullptr, row_start, row_len, row_ctx, row_slot};
    hipStream_t s = (hipStream_t)stream;
    const int64_t work = (int64_t)tokens * channels;
    hipLaunchKernelGGL(conv_silu_kernel, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, s, in, ldi, state, w, bias,
                       out, ldo, r, tokens, channels, taps);
    if (taps > 1) {
        const int64_t w2 = (int64_t)rows * channels;
        hipLaunchKernelGGL(conv_state_update_kernel, dim3((unsigned)((w2 + 255) / 256)), dim3(256), 0, s, in, ldi, state,
                           r, rows, channels, taps);
    }
    return check_launch();
}

int mv_conv_taps(const float* in, int64_t ldi, float* state, const float* w, float* out32, int64_t ld32, void* out_act,
                 int64_t ldoa, int add_input, const int32_t* tok_row, const int32_t* row_start, const int32_t* row_len,
                 const int32_t* row_ctx, const int32_t* row_slot, int tokens, int rows, int channels, int taps, int f32,
                 mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || rows < 0 || channels <= 0 || taps < 1 || taps > kMaxTaps) return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!in || (!state && taps > 1) || !w || (!out32 && !out_act) || ldi < channels || (out32 && ld32 < channels) ||
        (out_act && ldoa < channels) || !tok_row || !row_start || !row_len || !row_ctx || !row_slot)
        return MV_ERR_INVALID_ARG;
    StepRows r{tok_row, nullptr, row_start, row_len, row_ctx, row_slot};
    hipStream_t s = (hipStream_t)stream;
    const int64_t work = (int64_t)tokens * channels;
    const dim3 grid((unsigned)((work + 255) / 256));
    if (f32) hipLaunchKernelGGL(conv_taps_kernel<true>, grid, dim3(256), 0, s, in, ldi, state, w, out32, ld32, out_act, ldoa, add_input, r, tokens, channels, taps);
    else hipLaunchKernelGGL(conv_taps_kernel<false>, grid, dim3(256), 0, s, in, ldi, state, w, out32, ld32, out_act, ldoa, add_input, r, tokens, channels, taps);
    if (taps > 1) {
        const int64_t w2 = (int64_t)rows * channels;
        hipLaunchKernelGGL(conv_state_update_kernel, dim3((unsigned)((w2 + 255) / 256)), dim3(256), 0, s, in, ldi, state,
                           r, rows, channels, taps);
    }
    return check_launch();
}

int mv_conv_qkv_store(const float* in, int64_t ldi, float* state, const float* w, float* q, int64_t ldq, void* k_cache,
                      void* v_cache, const int32_t* tok_row, const int32_t* tok_pos, const int32_t* row_start,
                      const int32_t* row_len, const int32_t* row_ctx, const int32_t* row_slot,
                      const int32_t* block_table, int bt_stride, int page, int tokens, int rows, int cq, int ck, int cv,
                      int taps, int f32, mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || rows < 0 || cq <= 0 || ck <= 0 || cv <= 0 || taps < 0 || taps > kMaxTaps || page <= 0)
        return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    const int C = cq + ck + cv;
    if (!in || ldi < C || (taps > 0 && !w) || (taps > 1 && !state) || !q || ldq < cq || !k_cache || !v_cache ||
        !tok_row || !tok_pos || !row_start || !row_len || !row_ctx || !row_slot || !block_table)
        return MV_ERR_INVALID_ARG;
    StepRows r{tok_row, tok_pos, row_start, row_len, row_ctx, row_slot};
    PagedRows pr{tok_row, tok_pos, block_table, bt_stride, page};
    hipStream_t s = (hipStream_t)stream;
    const int64_t work = (int64_t)tokens * C;
    const dim3 grid((unsigned)((work + 255) / 256));
    const float* wk = taps > 0 ? w : nullptr;
    if (f32) hipLaunchKernelGGL(conv_qkv_store_kernel<true>, grid, dim3(256), 0, s, in, ldi, state, wk, q, ldq, k_cache, v_cache, r, pr, tokens, cq, ck, cv, taps);
    else hipLaunchKernelGGL(conv_qkv_store_kernel<false>, grid, dim3(256), 0, s, in, ldi, state, wk, q, ldq, k_cache, v_cache, r, pr, tokens, cq, ck, cv, taps);
    if (taps > 1) {
        const int64_t w2 = (int64_t)rows * C;
        hipLaunchKernelGGL(conv_state_update_kernel, dim3((unsigned)((w2 + 255) / 256)), dim3(256), 0, s, in, ldi, state,
                           r, rows, C, taps);
    }
    return check_launch();
}

int mv_softplus_decay(const float* raw, int64_t ld, const float* dt_bias, const float* a_log, float* gain,
                      float* decay, float* log_decay, int tokens, int heads, mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || heads <= 0) return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!raw || !dt_bias || !a_log || !gain || !decay || ld < heads) return MV_ERR_INVALID_ARG;
    hipLaunchKernelGGL(softplus_decay_kernel, dim3((tokens * heads + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                       raw, ld, dt_bias, a_log, gain, decay, log_decay, tokens, heads);
    return check_launch();
}

int mv_scan_outer(const float* q, int64_t ldq, int q_div, const float* k, int64_t ldk, int k_div, const float* v,
                  int64_t ldv, const float* decay, int64_t ld_decay, const float* gain, int64_t ld_gain,
                  const float* skip, float* state, float* out, int64_t ldo, const int32_t* row_start,
                  const int32_t* row_len, const int32_t* row_ctx, const int32_t* row_slot, int rows, int heads, int n,
                  int p, int max_len, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || heads <= 0 || n <= 0 || p <= 0 || q_div <= 0 || k_div <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!q || !k || !v || !decay || !state || !out || rows > 65535 || heads > 65535) return MV_ERR_INVALID_ARG;
    ScanArgs a;
    a.q = q; a.k = k; a.v = v; a.decay = decay; a.gain = gain; a.skip = skip;
    a.ldq = ldq; a.ldk = ldk; a.ldv = ldv; a.ld_decay = ld_decay; a.ld_gain = ld_gain; a.ldo = ldo;
    a.q_div = q_div; a.k_div = k_div; a.state = state; a.out = out;
    a.r = StepRows{nullptr, nullptr, row_start, row_len, row_ctx, row_slot};
    a.H = heads; a.n = n; a.p = p; a.max_len = max_len;
    a.ch_start = nullptr; a.ch_len = nullptr; a.ds = nullptr;
    a.pt = p % 64 == 0 ? 64 : (p % 32 == 0 ? 32 : 16);
    // a state too tall for 64 rows a thread: narrower column tiles leave more threads to share its rows
    while (a.pt > 16 && (n + 256 / a.pt - 1) / (256 / a.pt) > 64) a.pt /= 2;
    const int ns = 256 / a.pt, npt = (n + ns - 1) / ns;
    const dim3 grid((p + a.pt - 1) / a.pt, heads, rows);
    hipStream_t s = (hipStream_t)stream;
    if (npt <= 4) hipLaunchKernelGGL((scan_outer_kernel<4, false>), grid, dim3(256), 0, s, a);
    else if (npt <= 16) hipLaunchKernelGGL((scan_outer_kernel<16, false>), grid, dim3(256), 0, s, a);
    else if (npt <= 64) hipLaunchKernelGGL((scan_outer_kernel<64, false>), grid, dim3(256), 0, s, a);
    else return MV_ERR_UNSUPPORTED;
    return check_launch();
}

int mv_scan_gated(const float* q, int64_t ldq, const float* f, int64_t ldf, const float* v, int64_t ldv, float* state,
                  float* out, int64_t ldo, const int32_t* row_start, const int32_t* row_len, const int32_t* row_ctx,
                  const int32_t* row_slot, int rows, int heads, int n, int p, float* ds, float* cum,
                  const int32_t* ch_start, const int32_t* ch_len, const int32_t* row_ch0, const int32_t* row_nch,
                  int chunks, int max_len, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || heads <= 0 || n <= 0 || p <= 0 || chunks < 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!q || !f || !v || !state || !out || rows > 65535 || heads > 65535 || chunks > 65535) return MV_ERR_INVALID_ARG;
    if (ldq < (int64_t)heads * n || ldf < (int64_t)heads * n || ldv < (int64_t)heads * p || ldo < (int64_t)heads * p)
        return MV_ERR_INVALID_ARG;
    if (chunks > 0 && (!ds || !cum || !ch_start || !ch_len || !row_ch0 || !row_nch || max_len <= 0))
        return MV_ERR_INVALID_ARG;
    ScanArgs a;
    a.q = q; a.k = nullptr; a.v = v; a.decay = f; a.gain = nullptr; a.skip = nullptr;
    a.ldq = ldq; a.ldk = 0; a.ldv = ldv; a.ld_decay = ldf; a.ld_gain = 0; a.ldo = ldo;
    a.q_div = 1; a.k_div = 1; a.state = state; a.out = out;
    a.r = StepRows{nullptr, nullptr, row_start, row_len, row_ctx, row_slot};
    a.H = heads; a.n = n; a.p = p; a.max_len = chunks > 0 ? max_len : 0;
    a.ch_start = nullptr; a.ch_len = nullptr; a.ds = nullptr;
    hipStream_t s = (hipStream_t)stream;
    // rows of up to max_len tokens (all rows when nothing is cut into chunks): token by token from the slot's state
    for (int pass = 0; pass < (chunks > 0 ? 2 : 1); ++pass) {
        if (pass == 1) {
            a.ch_start = ch_start; a.ch_len = ch_len; a.ds = ds;
        }
        const int units = pass == 0 ? rows : chunks;
        a.pt = p % 64 == 0 ? 64 : (p % 32 == 0 ? 32 : 16);
        // a state too tall for 64 rows a thread: narrower column tiles leave more threads to share its rows; so do
        // launches that would not fill the chip otherwise (a few decoded tokens: the step is the state's traffic)
        while (a.pt > 16 && ((n + 256 / a.pt - 1) / (256 / a.pt) > 64 ||
                             (int64_t)((p + a.pt - 1) / a.pt) * heads * units < 2 * (int64_t)num_cus()))
            a.pt /= 2;
        const int ns = 256 / a.pt, npt = (n + ns - 1) / ns;
        if (npt > 64) return MV_ERR_UNSUPPORTED;
        const dim3 grid((p + a.pt - 1) / a.pt, heads, units);
        if (npt <= 4) hipLaunchKernelGGL((scan_outer_kernel<4, true>), grid, dim3(256), 0, s, a);
        else if (npt <= 16) hipLaunchKernelGGL((scan_outer_kernel<16, true>), grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL((scan_outer_kernel<64, true>), grid, dim3(256), 0, s, a);
    }
    if (chunks > 0) {
        const int width = heads * n;
        hipLaunchKernelGGL(gate_cumprod_kernel, dim3(chunks, (width + 255) / 256), dim3(256), 0, s, f, ldf, cum,
                           (int64_t)width, ch_start, ch_len, width);
        GatedChunkArgs g;
        g.q = q; g.cum = cum; g.ldq = ldq; g.ldc = width; g.ldo = ldo; g.state = state; g.out = out; g.ds = ds;
        g.ch_start = ch_start; g.ch_len = ch_len; g.row_ch0 = row_ch0; g.row_nch = row_nch; g.row_ctx = row_ctx;
        g.row_slot = row_slot; g.H = heads; g.n = n; g.p = p;
        hipLaunchKernelGGL(gated_carry_kernel, dim3((n * p + 255) / 256, heads, rows), dim3(256), 0, s, g);
        hipLaunchKernelGGL(gated_inter_kernel, dim3(chunks, heads, (p + 63) / 64), dim3(256), 0, s, g);
    }
    return check_launch();
}

int mv_gate_lower_bound(float* q, int64_t ldq, float* f, int64_t ldf, const float* bias, const float* lower,
                        int tokens, int n, mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!q || !f || !lower || ldq < n || ldf < n) return MV_ERR_INVALID_ARG;
    const int64_t total = (int64_t)tokens * n;
    hipLaunchKernelGGL(gate_lower_bound_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, q, ldq, f, ldf, bias, lower, tokens, n);
    return check_launch();
}

size_t mv_scan_chunked_lds_bytes(int n, int p) {
    const int n4 = (n + 3) & ~3;
    const size_t intra = (size_t)(2 * mv::kCh * (n4 + 1) + mv::kCh * (p + 1) + 3 * mv::kCh) * sizeof(float);
    const size_t inter = (size_t)(mv::kCh * (n4 + 1) + n4 * (p + 1)) * sizeof(float);
    return intra > inter ? intra : inter;
}

int mv_scan_chunked(const float* q, int64_t ldq, int q_div, const float* k, int64_t ldk, int k_div, const float* v,
                    int64_t ldv, const float* log_decay, int64_t ld_ld, const float* gain, int64_t ld_gain,
                    const float* skip, float* state, float* out, int64_t ldo, float* ds, float* lsum, float* atot,
                    const int32_t* ch_start, const int32_t* ch_len, const int32_t* row_ch0, const int32_t* row_nch,
                    const int32_t* row_ctx, const int32_t* row_slot, int chunks, int rows, int heads, int n, int p,
                    mv_stream_t stream) {
    using namespace mv;
    if (chunks < 0 || rows < 0 || heads <= 0 || n <= 0 || p <= 0 || q_div <= 0 || k_div <= 0) return MV_ERR_INVALID_ARG;
    if (chunks == 0) return MV_OK;
    if (!q || !k || !v || !log_decay || !state || !out || !ds || !lsum || !atot || !ch_start || !ch_len || !row_ch0 ||
        !row_nch || rows > 65535 || heads > 65535)
        return MV_ERR_INVALID_ARG;
    const int n4 = (n + 3) & ~3;
    const size_t lds = (size_t)(2 * kCh * (n4 + 1) + kCh * (p + 1) + 3 * kCh) * sizeof(float);
    const size_t lds2 = (size_t)(kCh * (n4 + 1) + n4 * (p + 1)) * sizeof(float);
    if (mv_scan_chunked_lds_bytes(n, p) > 150 * 1024) return MV_ERR_UNSUPPORTED;
    static LdsOptIn opt1, opt2;
    if (int rc = ensure_dynamic_lds((const void*)scan_chunk_intra_kernel, lds, opt1)) return rc;
    if (int rc = ensure_dynamic_lds((const void*)scan_chunk_inter_kernel, lds2, opt2)) return rc;
    ChunkArgs a;
    a.q = q; a.k = k; a.v = v; a.log_decay = log_decay; a.gain = gain; a.skip = skip;
    a.ldq = ldq; a.ldk = ldk; a.ldv = ldv; a.ld_ld = ld_ld; a.ld_gain = ld_gain; a.ldo = ldo;
    a.q_div = q_div; a.k_div = k_div; a.state = state; a.out = out; a.ds = ds; a.lsum = lsum; a.atot = atot;
    a.ch_start = ch_start; a.ch_len = ch_len; a.row_ch0 = row_ch0; a.row_nch = row_nch;
    a.r = StepRows{nullptr, nullptr, nullptr, nullptr, row_ctx, row_slot};
    a.H = heads; a.n = n; a.p = p;
    // heads that read the same q and k (a group) go four or two to a workgroup
    a.hb = (q_div == k_div && heads % q_div == 0) ? (q_div % 4 == 0 ? 4 : (q_div % 2 == 0 ? 2 : 1)) : 1;
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(scan_chunk_intra_kernel, dim3(chunks, heads / a.hb), dim3(256), lds, s, a);
    hipLaunchKernelGGL(scan_chunk_carry_kernel, dim3((n * p + 255) / 256, heads, rows), dim3(256), 0, s, a);
    hipLaunchKernelGGL(scan_chunk_inter_kernel, dim3(chunks, heads / a.hb), dim3(256), lds2, s, a);
    return check_launch();
}

int mv_rotary_pairs(float* x, int64_t ld, const double* inv_freq, const int32_t* tok_pos, int tokens, int heads,
                    int dim, int rot, float scale, mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || heads <= 0 || dim <= 0 || rot < 0 || rot > dim || rot % 2) return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!x || !tok_pos || (rot > 0 && !inv_freq) || ld < (int64_t)heads * dim) return MV_ERR_INVALID_ARG;
    const int64_t work = (int64_t)tokens * heads * (dim - rot / 2);
    hipLaunchKernelGGL(rotary_pairs_kernel, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x,
                       ld, inv_freq, tok_pos, tokens, heads, dim, rot, scale);
    return check_launch();
}

int mv_gated_group_norm(const float* y, int64_t ldy, const float* gate, int64_t ldg, const float* w, void* out,
                        int64_t ldo, int rows, int n, int groups, int gate_first, float eps, int f32,
                        mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0 || groups <= 0 || n % groups) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!y || !gate || !out || ldy < n || ldg < n || ldo < n) return MV_ERR_INVALID_ARG;
    const int64_t units = (int64_t)rows * groups;
    hipStream_t s = (hipStream_t)stream;
    if (n / groups >= 1024) {
        const dim3 wide((unsigned)units);
        if (f32) hipLaunchKernelGGL(gated_group_norm_wide_kernel<true>, wide, dim3(256), 0, s, y, ldy, gate, ldg, w, out, ldo, n, groups, gate_first, eps);
        else hipLaunchKernelGGL(gated_group_norm_wide_kernel<false>, wide, dim3(256), 0, s, y, ldy, gate, ldg, w, out, ldo, n, groups, gate_first, eps);
        return check_launch();
    }
    const dim3 grid((unsigned)((units + 3) / 4));
    if (f32) hipLaunchKernelGGL(gated_group_norm_kernel<true>, grid, dim3(256), 0, s, y, ldy, gate, ldg, w, out, ldo, rows, n, groups, gate_first, eps);
    else hipLaunchKernelGGL(gated_group_norm_kernel<false>, grid, dim3(256), 0, s, y, ldy, gate, ldg, w, out, ldo, rows, n, groups, gate_first, eps);
    return check_launch();
}

int mv_qk_unitnorm_store(float* qkv, int64_t ld, void* k_cache, void* v_cache, const int32_t* tok_row,
                         const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int page, int tokens,
                         int heads, int kv_heads, int d, int dv, float eps, int f32, mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || heads <= 0 || kv_heads <= 0 || d <= 0 || dv <= 0 || page <= 0 || heads % kv_heads)
        return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!qkv || !k_cache || !v_cache || !tok_row || !tok_pos || !block_table ||
        ld < (int64_t)(heads + kv_heads) * d + (int64_t)kv_heads * dv)
        return MV_ERR_INVALID_ARG;
    PagedRows pr{tok_row, tok_pos, block_table, bt_stride, page};
    const int64_t units = (int64_t)tokens * (heads + 2 * kv_heads);
    const dim3 grid((unsigned)((units + 3) / 4));
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(qk_unitnorm_store_kernel<true>, grid, dim3(256), 0, s, qkv, ld, k_cache, v_cache, pr, tokens, heads, kv_heads, d, dv, eps);
    else hipLaunchKernelGGL(qk_unitnorm_store_kernel<false>, grid, dim3(256), 0, s, qkv, ld, k_cache, v_cache, pr, tokens, heads, kv_heads, d, dv, eps);
    return check_launch();
}

int mv_qk_rotary_store(float* qk, int64_t ld, const float* q_bias, const float* k_bias, void* k_cache, void* v_cache,
                       const double* inv_freq, const int32_t* tok_row, const int32_t* tok_pos,
                       const int32_t* block_table, int bt_stride, int page, int tokens, int heads, int kv_heads, int d,
                       int rot, int adjacent, const float* act_in, int64_t lda, void* act_out, int64_t ldao, int act_n,
                       int act_kind, float act_limit, float act_slope, int f32, mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || heads <= 0 || kv_heads <= 0 || d <= 0 || page <= 0 || rot < 0 || rot > d || rot % 2)
        return MV_ERR_INVALID_ARG;
    if (act_in && (!act_out || act_n <= 0 || lda < 2 * (int64_t)act_n || ldao < act_n || act_kind < 0 || act_kind > 2))
        return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!qk || !k_cache || !v_cache || (rot > 0 && !inv_freq) || !tok_row || !tok_pos || !block_table ||
        ld < (int64_t)(heads + kv_heads) * d)
        return MV_ERR_INVALID_ARG;
    PagedRows pr{tok_row, tok_pos, block_table, bt_stride, page};
    // steps of many tokens: a wave takes eight heads of a token and forms the angles' sines and cosines once for them
    const int hpw = (int64_t)tokens * (heads + kv_heads) >= 8 * 1024 ? 8 : 1;
    const int64_t units = (int64_t)tokens * ((heads + kv_heads + hpw - 1) / hpw);
    const int64_t rot_blocks = (units + 3) / 4, act_blocks = act_in ? (int64_t)tokens * ((act_n + 255) / 256) : 0;
    if (rot_blocks + act_blocks > 0x7fffffff) return MV_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)(rot_blocks + act_blocks));
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(qk_rotary_store_kernel<true>, grid, dim3(256), 0, s, qk, ld, q_bias, k_bias, k_cache, v_cache, inv_freq, pr, tokens, heads, kv_heads, d, rot, adjacent, hpw, (unsigned)rot_blocks, act_in, lda, act_out, ldao, act_n, act_kind, act_limit, act_slope);
    else hipLaunchKernelGGL(qk_rotary_store_kernel<false>, grid, dim3(256), 0, s, qk, ld, q_bias, k_bias, k_cache, v_cache, inv_freq, pr, tokens, heads, kv_heads, d, rot, adjacent, hpw, (unsigned)rot_blocks, act_in, lda, act_out, ldao, act_n, act_kind, act_limit, act_slope);
    return check_launch();
}

int mv_window_attn_splits(int tokens, int heads, int kv_heads, int window, int keep_first) {
    using namespace mv;
    if (tokens <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads || window <= 0 || keep_first < 0) return 1;
    const int R = heads / kv_heads, ngrp = (R + kGrpMax - 1) / kGrpMax;
    const int64_t units = (int64_t)tokens * kv_heads * ngrp;
    const int64_t tiles = ((int64_t)window + keep_first) / 64 + 2;      // at most this many 64-key tiles a token
    int64_t want = (2 * (int64_t)num_cus() + units - 1) / units;         // about two workgroups a compute unit
    const int64_t most = (tiles + 3) / 4;                                // a wave should find a tile of its own
    if (want > most) want = most;
    if (want > 64) want = 64;
    return want < 1 ? 1 : (int)want;
}

int mv_window_attn(const float* q, int64_t ldq, const void* k_cache, const void* v_cache, void* out, int64_t ldo,
                   const int32_t* tok_row, const int32_t* tok_pos, const int32_t* block_table, int bt_stride,
                   int page, const float* slopes, int tokens, int heads, int kv_heads, int d, int dv, float scale,
                   int window, int f32, const int32_t* row_len, const int32_t* ch_start, const int32_t* ch_len,
                   int chunks, int max_len, int keep_first, const float* sinks, float* part, int splits,
                   int short_tokens, mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || heads <= 0 || kv_heads <= 0 || d <= 0 || dv <= 0 || page <= 0 || window <= 0 ||
        heads % kv_heads || keep_first < 0)
        return MV_ERR_INVALID_ARG;
    if (dv > 64 * kMaxVC || d > 4096) return MV_ERR_UNSUPPORTED;
    if (tokens == 0) return MV_OK;
    if (!q || !k_cache || !v_cache || !out || !tok_row || !tok_pos || !block_table) return MV_ERR_INVALID_ARG;
    PagedRows pr{tok_row, tok_pos, block_table, bt_stride, page};
    const int64_t units = (int64_t)tokens * heads;
    if (units > 0x7fffffff) return MV_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)units);
    hipStream_t s = (hipStream_t)stream;
    // rows of more than max_len tokens, cut into the chunks of the table: the tiled matrix-core kernel, where
    // the shapes are among those it is built for (bf16, 64-token pages, 16-byte rows)
    int skip_len = 0;
    if (!f32 && chunks > 0 && max_len > 0 && row_len && ch_start && ch_len && page == 64 && ldq % 4 == 0 &&
        ldo % 4 == 0 && aligned16(q) && aligned16(k_cache) && aligned16(v_cache) && (reinterpret_cast<uintptr_t>(out) & 7) == 0) {
        const dim3 tg(chunks, heads);
#define MV_WA_TILE(KS_, CT_)                                                                                         \
    hipLaunchKernelGGL((window_attn_tile_kernel<KS_, CT_>), tg, dim3(256), 0, s, q, ldq, (const uint16_t*)k_cache,      \
                       (const uint16_t*)v_cache, (uint16_t*)out, ldo, pr, ch_start, ch_len, slopes, heads, kv_heads, scale, \
                       window, keep_first, sinks);                                                                                    \
    skip_len = max_len
        if (d == 64 && dv == 64) { MV_WA_TILE(2, 4); }
        else if (d == 96 && dv == 96) { MV_WA_TILE(3, 6); }
        else if (d == 128 && dv == 128) { MV_WA_TILE(4, 8); }
        else if (d == 128 && dv == 64) { MV_WA_TILE(4, 4); }
        else if (d == 64 && dv == 128) { MV_WA_TILE(2, 8); }
        else if (d == 32 && dv == 32) { MV_WA_TILE(1, 2); }
#undef MV_WA_TILE
        // every row of the step was long enough for the tiles: nothing is left for the per-token forms
        if (skip_len > 0 && short_tokens == 0) return check_launch();
    }
    // with a place for the splits' pieces: the kernel that shares every key among the query heads of its key/value
    // head and cuts the keys over several workgroups
    if (part && splits >= 1) {
        const int R = heads / kv_heads, ngrp = (R + kGrpMax - 1) / kGrpMax, top = R < kGrpMax ? R : kGrpMax;
        const int rt = top <= 1 ? 1 : top <= 2 ? 2 : top <= 4 ? 4 : 8;
        const int vecw = f32 ? 4 : 8;
        const int vec = dv % vecw == 0 && dv / vecw <= 64 && aligned16(v_cache);
        const size_t glds = ((size_t)rt * d + 4 * rt * 64 + 4 * (size_t)rt * dv + 8 * rt) * sizeof(float);
        if (glds <= 64 * 1024 && d % 4 == 0 && ldq % 4 == 0 && aligned16(q) && (f32 || d % 8 != 0 || aligned16(k_cache))) {
            const dim3 gg((unsigned)(tokens * kv_heads * ngrp), splits);
#define MV_WA_GROUP(F32_, RT_)                                                                                         \
    hipLaunchKernelGGL((window_attn_group_kernel<F32_, RT_>), gg, dim3(256), glds, s, q, ldq, k_cache, v_cache, out, ldo, \
                       part, pr, slopes, sinks, heads, kv_heads, d, dv, scale, window, keep_first, row_len, skip_len,   \
                       splits, vec)
            if (f32) {
                if (rt == 1) MV_WA_GROUP(true, 1); else if (rt == 2) MV_WA_GROUP(true, 2);
                else if (rt == 4) MV_WA_GROUP(true, 4); else MV_WA_GROUP(true, 8);
            } else {
                if (rt == 1) MV_WA_GROUP(false, 1); else if (rt == 2) MV_WA_GROUP(false, 2);
                else if (rt == 4) MV_WA_GROUP(false, 4); else MV_WA_GROUP(false, 8);
            }
#undef MV_WA_GROUP
            if (splits > 1) {
                if (f32) hipLaunchKernelGGL(window_attn_merge_kernel<true>, grid, dim3(64), 0, s, part, out, ldo, tok_row, sinks, heads, dv, splits, row_len, skip_len);
                else hipLaunchKernelGGL(window_attn_merge_kernel<false>, grid, dim3(64), 0, s, part, out, ldo, tok_row, sinks, heads, dv, splits, row_len, skip_len);
            }
            return check_launch();
        }
    }
    // few (token, head) pairs and a window of many tiles: sixteen waves share it
    const bool wide = units <= 2 * num_cus() && window > 256;
    const int nw = wide ? 16 : 4;
    const size_t lds = (size_t)(d + 64 * nw + 2 * nw + nw * dv) * sizeof(float);
    if (lds > 64 * 1024) return MV_ERR_UNSUPPORTED;
    if (wide) {
        if (f32) hipLaunchKernelGGL((window_attn_kernel<true, 16>), grid, dim3(1024), lds, s, q, ldq, k_cache, v_cache, out, ldo, pr, slopes, tokens, heads, kv_heads, d, dv, scale, window, row_len, skip_len, keep_first, sinks);
        else hipLaunchKernelGGL((window_attn_kernel<false, 16>), grid, dim3(1024), lds, s, q, ldq, k_cache, v_cache, out, ldo, pr, slopes, tokens, heads, kv_heads, d, dv, scale, window, row_len, skip_len, keep_first, sinks);
    } else {
        if (f32) hipLaunchKernelGGL((window_attn_kernel<true, 4>), grid, dim3(256), lds, s, q, ldq, k_cache, v_cache, out, ldo, pr, slopes, tokens, heads, kv_heads, d, dv, scale, window, row_len, skip_len, keep_first, sinks);
        else hipLaunchKernelGGL((window_attn_kernel<false, 4>), grid, dim3(256), lds, s, q, ldq, k_cache, v_cache, out, ldo, pr, slopes, tokens, heads, kv_heads, d, dv, scale, window, row_len, skip_len, keep_first, sinks);
    }
    return check_launch();
}

}  // extern "C"
