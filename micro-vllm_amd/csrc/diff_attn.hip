// Differential attention over paged keys and values: every query head carries TWO softmax maps (two query vectors
// of d dimensions, scored against the two key vectors of its key/value head) that weigh the SAME values; what
// leaves the head is  o = a1 - lambda a2,  divided by its root mean square over the head's dv values, times
// `out_scale`, times sigmoid(gate) of one number per (token, head).  No positions enter the scores; the mask is
// causal.  With `cap` > 0 a score passes  cap * tanh(score / cap)  before the softmax.
//
// Pages: a token's key row holds its kv heads' pairs of key vectors, [G][2][d]; its value row [G][dv].  Query head h
// reads key/value head h / (H / G); q is [T][H][2][d] in fp32.  Both maps of a head are formed from ONE read of each
// key row and ONE read of each value row.
//
//   diff_attn_kernel       a workgroup per (token, head); its 4 or 16 waves take the visible keys in tiles of 64, a
//                          lane scoring one key for both maps, then lanes own value columns; the waves' partial
//                          softmaxes meet in LDS, where the head's difference, norm and gate are applied.  Serves
//                          decoded tokens, short rows, fp32 and every head shape.
//   diff_attn_tile_kernel  a prompt's portion in bf16 on the matrix cores: a workgroup per (64 consecutive tokens of
//                          a row, head), a wave per 16 of them; a page is staged once in LDS (both key vectors and
//                          the values as pairs of neighbouring keys), q.k on v_mfma_f32_16x16x32_bf16, cap, mask and
//                          softmax in fp32 per lane, P.V with every fp32 weight split exactly into three bf16
//                          numbers (three bf16 matrix instructions with fp32 accumulators form the products an fp32
//                          one would).
// Scores, weights, the difference and the norm are fp32; the activation type (bf16 or fp32) concerns the pages and
// the output only.
#include "common.h"

namespace mv {

template <bool F32> struct ActD;
template <> struct ActD<true> {
    typedef float T;
    static __device__ __forceinline__ float ld(const float* p) { return *p; }
    static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct ActD<false> {
    typedef uint16_t T;
    static __device__ __forceinline__ float ld(const uint16_t* p) { return bf16_bits_to_f32(*p); }
    static __device__ __forceinline__ void st(uint16_t* p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }
};

struct DiffPages {
    const int* tok_row;
    const int* tok_pos;
    const int* block_table;
    int bt_stride, page;
};

struct DiffConsts {
    float scale, cap, lambda, out_scale, eps;
};

constexpr int kDiffVC = 4;  // value columns per lane: dv <= 256

__device__ __forceinline__ float capped(float s, float cap) { return cap > 0.f ? cap * tanhf(s / cap) : s; }

template <bool F32, int NW>
__global__ __launch_bounds__(64 * NW) void diff_attn_kernel(const float* q, int64_t ldq, const void* kc_,
                                                            const void* vc_, void* out_, int64_t ldo,
                                                            const float* gate, int64_t ldg, DiffPages pr, int H, int G,
                                                            int d, int dv, DiffConsts k, const int* row_len,
                                                            int max_len) {
    typedef typename ActD<F32>::T T_;
    extern __shared__ float lds[];
    if (max_len > 0 && row_len[pr.tok_row[blockIdx.x / H]] > max_len) return;   // the tile kernel's rows
    const T_* kc = (const T_*)kc_;
    const T_* vc = (const T_*)vc_;
    T_* out = (T_*)out_;
    const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float* qs = lds;                         // [2 d]
    float* ps = lds + 2 * d + wv * 128;      // [NW][2][64]
    float* mm = lds + 2 * d + 128 * NW;      // [NW][2]
    float* ll = mm + 2 * NW;                 // [NW][2]
    float* aa = ll + 2 * NW;                 // [NW][2][dv]
    const int t = blockIdx.x / H, h = blockIdx.x % H, g = h / (H / G);
    const int pos = pr.tok_pos[t];
    const int* bt = pr.block_table + (int64_t)pr.tok_row[t] * pr.bt_stride;
    for (int c = threadIdx.x; c < 2 * d; c += 64 * NW) qs[c] = q[(int64_t)t * ldq + (int64_t)h * 2 * d + c];
    __syncthreads();
    float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
    float acc[2][kDiffVC] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    for (int j0 = 64 * wv; j0 <= pos; j0 += 64 * NW) {
        const int j = j0 + lane;
        float s[2] = {-INFINITY, -INFINITY};
        if (j <= pos) {
            const int pg = bt[j / pr.page];
            const T_* kr = kc + (((int64_t)pg * pr.page + j % pr.page) * G + g) * 2 * d;
#pragma unroll
            for (int mp = 0; mp < 2; ++mp) {
                const T_* km = kr + mp * d;
                const float* qm = qs + mp * d;
                float dot = 0.f;
                if (!F32 && (d & 7) == 0) {
                    for (int c = 0; c < d; c += 8) {
                        const uint4 kv = ld16(km + c);
                        const uint32_t w[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            dot = fmaf(qm[c + 2 * e], bf16_lo(w[e]), dot);
                            dot = fmaf(qm[c + 2 * e + 1], bf16_hi(w[e]), dot);
                        }
                    }
                } else {
                    for (int c = 0; c < d; ++c) dot = fmaf(qm[c], ActD<F32>::ld(km + c), dot);
                }
                s[mp] = capped(dot * k.scale, k.cap);
            }
        }
        float corr[2];
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int mp = 0; mp < 2; ++mp) {
            const float mn = fmaxf(m[mp], wave_max(s[mp]));
            const float pj = j <= pos ? expf(s[mp] - mn) : 0.f;
            corr[mp] = expf(m[mp] - mn);       // m = -inf on the wave's first tile: exp(-inf) = 0
            l[mp] = l[mp] * corr[mp] + wave_sum(pj);
            m[mp] = mn;
            ps[mp * 64 + lane] = pj;
#pragma unroll
            for (int ci = 0; ci < kDiffVC; ++ci) acc[mp][ci] *= corr[mp];
        }
        __builtin_amdgcn_wave_barrier();
        const int cnt = pos - j0 + 1 < 64 ? pos - j0 + 1 : 64;
        // eight value rows at a time, their loads in flight together; each serves both maps
        for (int jj = 0; jj < cnt; jj += 8) {
            float p1[8], p2[8];
            const T_* vr[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const bool ok = jj + u < cnt;
                const int jk = ok ? j0 + jj + u : j0;
                const int pg = bt[jk / pr.page];
                vr[u] = vc + (((int64_t)pg * pr.page + jk % pr.page) * G + g) * dv;
                p1[u] = ok ? ps[jj + u] : 0.f;
                p2[u] = ok ? ps[64 + jj + u] : 0.f;
            }
#pragma unroll
            for (int ci = 0; ci < kDiffVC; ++ci) {
                const int c = lane + ci * 64;
                if (c < dv) {
                    float x[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) x[u] = ActD<F32>::ld(vr[u] + c);
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        acc[0][ci] = fmaf(p1[u], x[u], acc[0][ci]);
                        acc[1][ci] = fmaf(p2[u], x[u], acc[1][ci]);
                    }
                }
            }
        }
    }
    if (lane == 0) {
        mm[2 * wv] = m[0];
        mm[2 * wv + 1] = m[1];
        ll[2 * wv] = l[0];
        ll[2 * wv + 1] = l[1];
    }
#pragma unroll
    for (int ci = 0; ci < kDiffVC; ++ci) {
        const int c = lane + ci * 64;
        if (c < dv) {
            aa[(2 * wv) * dv + c] = acc[0][ci];
            aa[(2 * wv + 1) * dv + c] = acc[1][ci];
        }
    }
    __syncthreads();
    if (wv == 0) {
        float o[kDiffVC] = {0.f, 0.f, 0.f, 0.f};
        float a[2][kDiffVC];
#pragma unroll
        for (int mp = 0; mp < 2; ++mp) {
            float M = mm[mp];                              // wave 0 always has a key: finite
#pragma unroll
            for (int w = 1; w < NW; ++w) M = fmaxf(M, mm[2 * w + mp]);
            float L = 0.f;
            float w4[NW];
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                w4[w] = expf(mm[2 * w + mp] - M);          // a wave without keys: exp(-inf) = 0
                L = fmaf(ll[2 * w + mp], w4[w], L);
            }
#pragma unroll
            for (int ci = 0; ci < kDiffVC; ++ci) {
                const int c = lane + ci * 64;
                float v = 0.f;
                if (c < dv) {
#pragma unroll
                    for (int w = 0; w < NW; ++w) v = fmaf(aa[(2 * w + mp) * dv + c], w4[w], v);
                }
                a[mp][ci] = v / L;
            }
        }
        float ss = 0.f;
#pragma unroll
        for (int ci = 0; ci < kDiffVC; ++ci) {
            o[ci] = a[0][ci] - k.lambda * a[1][ci];        // columns past dv are zero on both sides
            ss += o[ci] * o[ci];
        }
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)dv + k.eps);
        const float gt = gate ? 1.0f / (1.0f + expf(-gate[(int64_t)t * ldg + h])) : 1.0f;
        const float f = inv * k.out_scale * gt;
#pragma unroll
        for (int ci = 0; ci < kDiffVC; ++ci) {
            const int c = lane + ci * 64;
            if (c < dv) ActD<F32>::st(out + (int64_t)t * ldo + (int64_t)h * dv + c, o[ci] * f);
        }
    }
}

typedef __attribute__((ext_vector_type(8))) __bf16 da_bf16x8_t;

// KS = d / 32, CT = dv / 16.  Accumulators of a lane after the score products: S[key 16 nt + 4 (lane / 16) + j][query
// lane % 16]; they serve as the second operand of the P.V products where they lie (the contraction index of the
// instruction is only a label; the value operand is gathered to match).
template <int KS, int CT>
__global__ __launch_bounds__(256) void diff_attn_tile_kernel(const float* q, int64_t ldq, const uint16_t* kc,
                                                             const uint16_t* vc, uint16_t* out, int64_t ldo,
                                                             const float* gate, int64_t ldg, DiffPages pr,
                                                             const int* ch_start, const int* ch_len, int H, int G,
                                                             DiffConsts k) {
    constexpr int D = KS * 32, DV = CT * 16, SK = 2 * D + 8, SV = DV + 8;
    __shared__ __attribute__((aligned(16))) uint16_t Ks[64][SK];
    __shared__ __attribute__((aligned(16))) uint32_t Vp[32][SV];   // dword [i][c] = V[2i][c] | V[2i+1][c] << 16
    const int ch = blockIdx.x, h = blockIdx.y, g = h / (H / G);
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, r = lane & 15, qd = lane >> 4;
    const int start = ch_start[ch], len = ch_len[ch];
    const int* bt = pr.block_table + (int64_t)pr.tok_row[start] * pr.bt_stride;
    const int p0 = pr.tok_pos[start];            // positions run on from here within the chunk
    const int myq = 16 * wv + r;
    const bool qok = myq < len;
    const int qpos = p0 + myq;
    da_bf16x8_t qf[2][KS];
    {
        const float* qp = q + (int64_t)(start + (qok ? myq : 0)) * ldq + (int64_t)h * 2 * D + 8 * qd;
#pragma unroll
        for (int mp = 0; mp < 2; ++mp)
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) {
                const float4 a = *reinterpret_cast<const float4*>(qp + mp * D + 32 * kk);
                const float4 b = *reinterpret_cast<const float4*>(qp + mp * D + 32 * kk + 4);
                const uint4 pk = make_uint4(pack_bf16x2(a.x, a.y), pack_bf16x2(a.z, a.w), pack_bf16x2(b.x, b.y),
                                            pack_bf16x2(b.z, b.w));
                qf[mp][kk] = __builtin_bit_cast(da_bf16x8_t, pk);
            }
    }
    float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
    f32x4_t o[2][CT];
#pragma unroll
    for (int mp = 0; mp < 2; ++mp)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) o[mp][ct] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const int khi = p0 + len - 1;
    const int wq_hi = p0 + 16 * wv + 15;          // this wave's last query position
    constexpr float kLog2e = 1.4426950408889634f;  // e^x as 2^(x log2 e) on the hardware's exp2
    for (int kt = 0; kt <= khi / 64; ++kt) {
        const int kbase = kt * 64;
        const int64_t pgrow = (int64_t)bt[kt] * 64;
        __syncthreads();
        for (int i = tid; i < 64 * (2 * D / 8); i += 256) {
            const int rr = i / (2 * D / 8), cc = i % (2 * D / 8);
            st16(&Ks[rr][cc * 8], ld16(kc + ((pgrow + rr) * G + g) * 2 * D + cc * 8));
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
        if (kbase > wq_hi) continue;               // nothing of this tile is visible to the wave
#pragma unroll
        for (int mp = 0; mp < 2; ++mp) {
            f32x4_t sc[4];
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
                sc[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < KS; ++kk) {
                    const da_bf16x8_t kf =
                        __builtin_bit_cast(da_bf16x8_t, ld16(&Ks[16 * nt + r][mp * D + 32 * kk + 8 * qd]));
                    sc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[mp][kk], sc[nt], 0, 0, 0);
                }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int kpos = kbase + 16 * nt + 4 * qd + j;
                    const bool ok = qok && kpos <= qpos;
                    const float v = ok ? capped(sc[nt][j] * k.scale, k.cap) : -INFINITY;
                    sc[nt][j] = v;
                    mx = fmaxf(mx, v);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float mn = fmaxf(m[mp], mx);
            const float corr = m[mp] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m[mp] - mn) * kLog2e);
            float psum = 0.f;
#pragma unroll
            for (int nt = 0; nt < 4; ++nt)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float pv = sc[nt][j] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((sc[nt][j] - mn) * kLog2e);
                    sc[nt][j] = pv;
                    psum += pv;
                }
            psum += __shfl_xor(psum, 16, 64);
            psum += __shfl_xor(psum, 32, 64);
            l[mp] = l[mp] * corr + psum;
            m[mp] = mn;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) o[mp][ct] *= corr;
            // an fp32 weight is the exact sum of three bf16 numbers (its leading 8, next 8 and last 8 mantissa bits,
            // each cut off, not rounded); slot (qd, e) of both operands stands for key 32 kb + 16 (e / 4) + 4 qd + e % 4
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                uint32_t hi[4], mid[4], lo[4];
#pragma unroll
                for (int e2 = 0; e2 < 4; ++e2) {
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
                const da_bf16x8_t ph = __builtin_bit_cast(da_bf16x8_t, make_uint4(hi[0], hi[1], hi[2], hi[3]));
                const da_bf16x8_t pm = __builtin_bit_cast(da_bf16x8_t, make_uint4(mid[0], mid[1], mid[2], mid[3]));
                const da_bf16x8_t pl = __builtin_bit_cast(da_bf16x8_t, make_uint4(lo[0], lo[1], lo[2], lo[3]));
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    uint32_t vw[4];
#pragma unroll
                    for (int e2 = 0; e2 < 4; ++e2)     // keys k0, k0 + 1 with k0 = 32 kb + 16 (e2 / 2) + 4 qd + 2 (e2 % 2)
                        vw[e2] = Vp[16 * kb + 8 * (e2 / 2) + 2 * qd + (e2 % 2)][16 * ct + r];
                    const da_bf16x8_t vf = __builtin_bit_cast(da_bf16x8_t, make_uint4(vw[0], vw[1], vw[2], vw[3]));
                    o[mp][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, ph, o[mp][ct], 0, 0, 0);
                    o[mp][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pm, o[mp][ct], 0, 0, 0);
                    o[mp][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pl, o[mp][ct], 0, 0, 0);
                }
            }
        }
    }
    // a lane holds columns 16 ct + 4 qd + j of query r: the head's sum of squares is spread over the four lanes
    // r, r + 16, r + 32, r + 48
    const float i1 = qok ? 1.0f / l[0] : 0.f, i2 = qok ? k.lambda / l[1] : 0.f;
    float ss = 0.f;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float v = o[0][ct][j] * i1 - o[1][ct][j] * i2;
            o[0][ct][j] = v;
            ss += v * v;
        }
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    if (qok) {
        const float gt = gate ? 1.0f / (1.0f + expf(-gate[(int64_t)(start + myq) * ldg + h])) : 1.0f;
        const float f = k.out_scale * gt / sqrtf(ss / (float)DV + k.eps);
        uint16_t* op = out + (int64_t)(start + myq) * ldo + (int64_t)h * DV + 4 * qd;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            uint2 w;
            w.x = pack_bf16x2(o[0][ct][0] * f, o[0][ct][1] * f);
            w.y = pack_bf16x2(o[0][ct][2] * f, o[0][ct][3] * f);
            *reinterpret_cast<uint2*>(op + 16 * ct) = w;
        }
    }
}

}  // namespace mv

extern "C" {

int mv_diff_attn(const float* q, int64_t ldq, const void* k_cache, const void* v_cache, void* out, int64_t ldo,
                 const float* gate, int64_t ldg, const int32_t* tok_row, const int32_t* tok_pos,
                 const int32_t* block_table, int bt_stride, int page, int tokens, int heads, int kv_heads, int d, int dv,
                 float scale, float cap, float lambda, float out_scale, float eps, int f32, const int32_t* row_len,
                 const int32_t* ch_start, const int32_t* ch_len, int chunks, int max_len, int short_tokens,
                 mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || heads <= 0 || kv_heads <= 0 || d <= 0 || dv <= 0 || page <= 0 || heads % kv_heads || cap < 0.f)
        return MV_ERR_INVALID_ARG;
    if (dv > 64 * kDiffVC || d > 2048) return MV_ERR_UNSUPPORTED;
    if (tokens == 0) return MV_OK;
    if (!q || !k_cache || !v_cache || !out || !tok_row || !tok_pos || !block_table || ldq < (int64_t)heads * 2 * d ||
        ldo < (int64_t)heads * dv || (gate && ldg < heads))
        return MV_ERR_INVALID_ARG;
    const DiffPages pr{tok_row, tok_pos, block_table, bt_stride, page};
    const DiffConsts k{scale, cap, lambda, out_scale, eps};
    const int64_t units = (int64_t)tokens * heads;
    if (units > 0x7fffffff) return MV_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    // rows of more than max_len tokens, cut into the chunks of the table: the matrix-core kernel, where the shapes
    // are among those it is built for (bf16, 64-token pages, 16-byte rows)
    int skip_len = 0;
    if (!f32 && chunks > 0 && max_len > 0 && row_len && ch_start && ch_len && page == 64 && ldq % 4 == 0 &&
        ldo % 4 == 0 && aligned16(q) && aligned16(k_cache) && aligned16(v_cache) &&
        (reinterpret_cast<uintptr_t>(out) & 7) == 0 && heads <= 65535) {
        const dim3 tg(chunks, heads);
#define MV_DA_TILE(KS_, CT_)                                                                                        \
    hipLaunchKernelGGL((diff_attn_tile_kernel<KS_, CT_>), tg, dim3(256), 0, s, q, ldq, (const uint16_t*)k_cache,    \
                       (const uint16_t*)v_cache, (uint16_t*)out, ldo, gate, ldg, pr, ch_start, ch_len, heads,       \
                       kv_heads, k);                                                                                \
    skip_len = max_len
        if (d == 64 && dv == 128) { MV_DA_TILE(2, 8); }
        else if (d == 64 && dv == 64) { MV_DA_TILE(2, 4); }
        else if (d == 32 && dv == 64) { MV_DA_TILE(1, 4); }
        else if (d == 32 && dv == 32) { MV_DA_TILE(1, 2); }
        else if (d == 128 && dv == 128) { MV_DA_TILE(4, 8); }
#undef MV_DA_TILE
        if (skip_len > 0 && short_tokens == 0) return check_launch();
    }
    // few (token, head) pairs: sixteen waves share a token's keys
    const bool wide = units <= 2 * (int64_t)num_cus();
    const int nw = wide ? 16 : 4;
    const size_t lds = (size_t)(2 * d + 128 * nw + 4 * nw + 2 * nw * dv) * sizeof(float);
    if (lds > 64 * 1024) return MV_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)units);
    if (wide) {
        if (f32) hipLaunchKernelGGL((diff_attn_kernel<true, 16>), grid, dim3(1024), lds, s, q, ldq, k_cache, v_cache, out, ldo, gate, ldg, pr, heads, kv_heads, d, dv, k, row_len, skip_len);
        else hipLaunchKernelGGL((diff_attn_kernel<false, 16>), grid, dim3(1024), lds, s, q, ldq, k_cache, v_cache, out, ldo, gate, ldg, pr, heads, kv_heads, d, dv, k, row_len, skip_len);
    } else {
        if (f32) hipLaunchKernelGGL((diff_attn_kernel<true, 4>), grid, dim3(256), lds, s, q, ldq, k_cache, v_cache, out, ldo, gate, ldg, pr, heads, kv_heads, d, dv, k, row_len, skip_len);
        else hipLaunchKernelGGL((diff_attn_kernel<false, 4>), grid, dim3(256), lds, s, q, ldq, k_cache, v_cache, out, ldo, gate, ldg, pr, heads, kv_heads, d, dv, k, row_len, skip_len);
    }
    return check_launch();
}

}  // extern "C"
