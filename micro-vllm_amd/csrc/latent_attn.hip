// Attention over a cached LATENT: every token keeps one normed vector c (R values) and one rotated key part
// (r values) shared by all heads, in pages of [R + r].  A head's unrotated key W_uk c and value W_uv c are
// never formed: the query is carried into the latent space (q_abs = W_uk^T q_unrotated, a per-head
// product done by mv_linear_heads), scores are q_abs . c + q_rot . k_rot, the weighted sum of the cached c
// comes out of the kernel and W_uv is applied to it afterwards (again per head).  So all heads of a token
// read the same R + r numbers per key, and the values are the first R of them.
//
//   latent_prep   c = unit-RMS(first R of the down-projection) * w into the page, the last r rotated by
//                 position into the page; q's rotated part rotated into the query buffer [H, R + r] at
//                 column R, q's unrotated part copied in the activation type for the per-head product.
//                 Rotation over the first `rot` of the r dimensions, pairs (2i, 2i+1) or (i, i + rot/2).
//   latent_attn   softmax over the visible keys (all j <= i, or the last `window` of them), optionally with
//                 a per-head sink: exp(sink_h) joins the denominator and carries no value.
// Scores, weights, norms, angles: fp32 (angles formed in fp64 from an fp64 frequency table).
#include "common.h"

namespace mv {

template <bool F32> struct ActL;
template <> struct ActL<true> {
    typedef float T;
    static __device__ __forceinline__ float ld(const float* p) { return *p; }
    static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct ActL<false> {
    typedef uint16_t T;
    static __device__ __forceinline__ float ld(const uint16_t* p) { return bf16_bits_to_f32(*p); }
    static __device__ __forceinline__ void st(uint16_t* p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }
};

struct LatentPages {
    const int* tok_row;
    const int* tok_pos;
    const int* block_table;
    int bt_stride, page;
};

// pair (a, b) of a rotated vector of `rot` dimensions: index of its two members
__device__ __forceinline__ void rot_pair(int i, int rot, int interleaved, int& a, int& b) {
    if (interleaved) {
        a = 2 * i;
        b = 2 * i + 1;
    } else {
        a = i;
        b = i + rot / 2;
    }
}

template <bool F32>
__global__ __launch_bounds__(256) void latent_prep_kernel(const float* dkv, int64_t ldkv, const float* wn, float eps,
                                                          void* cache_, const float* q, int64_t ldq, void* qn_,
                                                          int64_t ldqn, float* qabs, int64_t ldqa,
                                                          const double* inv_freq, LatentPages pr, int H, int d, int r,
                                                          int R, int rot, int interleaved) {
    typedef typename ActL<F32>::T T_;
    __shared__ float red[4];
    T_* cache = (T_*)cache_;
    T_* qn = (T_*)qn_;
    const int t = blockIdx.x, tid = threadIdx.x;
    const int pos = pr.tok_pos[t];
    const int pg = pr.block_table[(int64_t)pr.tok_row[t] * pr.bt_stride + pos / pr.page];
    T_* dst = cache + ((int64_t)pg * pr.page + pos % pr.page) * (R + r);
    const float* row = dkv + (int64_t)t * ldkv;
    float ss = 0.f;
    for (int c = tid; c < R; c += 256) ss += row[c] * row[c];
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)R + eps);
    if (pg >= 0)
        for (int c = tid; c < R; c += 256) ActL<F32>::st(dst + c, (row[c] * inv) * wn[c]);
    const int half = rot / 2;
    // the shared key part and the heads' query parts: unit u = 0 is the key, u = 1 + h a head
    for (int i = tid; i < (H + 1) * (r - half); i += 256) {
        const int u = i / (r - half), j = i % (r - half);
        const float* src = u == 0 ? row + R : q + (int64_t)t * ldq + (int64_t)(u - 1) * (d + r) + d;
        float o0, o1 = 0.f;
        int a, b = -1;
        if (j < half) {
            rot_pair(j, rot, interleaved, a, b);
            const double ang = (double)pos * inv_freq[j];
            const float cs = (float)cos(ang), sn = (float)sin(ang);
            o0 = src[a] * cs - src[b] * sn;
            o1 = src[b] * cs + src[a] * sn;
        } else {
            a = rot + (j - half);   // passes unchanged
            o0 = src[a];
        }
        if (u == 0) {
            if (pg >= 0) {
                ActL<F32>::st(dst + R + a, o0);
                if (b >= 0) ActL<F32>::st(dst + R + b, o1);
            }
        } else {
            float* qa = qabs + (int64_t)t * ldqa + (int64_t)(u - 1) * (R + r) + R;
            qa[a] = o0;
            if (b >= 0) qa[b] = o1;
        }
    }
    for (int i = tid; i < H * d; i += 256) {
        const int h = i / d, c = i % d;
        ActL<F32>::st(qn + (int64_t)t * ldqn + i, q[(int64_t)t * ldq + (int64_t)h * (d + r) + c]);
    }
}

// One workgroup per (token, group of up to HG heads).  Its NW waves take the visible keys in tiles of 64 in
// turn: a lane scores ONE key for all heads of the group (the key's R + r numbers are read once, the
// queries lie in LDS), the wave forms max and sum of the tile per head, then lanes own value columns and
// add the tile's weighted latents for every head from one read of each.  The waves' partial softmaxes are
// merged in a fixed order.  Serves prompts' portions and single decoded tokens alike.
template <bool F32, int NW, int HG, int VC>
__global__ __launch_bounds__(64 * NW) void latent_attn_kernel(const float* q, int64_t ldq, const void* cache_,
                                                              void* out_, int64_t ldo, LatentPages pr,
                                                              const float* sinks, int H, int R, int r, float scale,
                                                              int window, const int* row_len, int max_len) {
    typedef typename ActL<F32>::T T_;
    extern __shared__ float lds[];
    {   // rows of more than max_len tokens belong to the tile kernel
        const int groups_ = (H + HG - 1) / HG;
        if (max_len > 0 && row_len[pr.tok_row[blockIdx.x / groups_]] > max_len) return;
    }
    const T_* cache = (const T_*)cache_;
    T_* out = (T_*)out_;
    const int d = R + r;
    const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int groups = (H + HG - 1) / HG;
    const int t = blockIdx.x / groups, h0 = (blockIdx.x % groups) * HG;
    const int nh = H - h0 < HG ? H - h0 : HG;
    float* qs = lds;                                  // [HG][d]
    float* ps = lds + HG * d + wv * HG * 64;          // [NW][HG][64]
    float* mm = lds + HG * d + NW * HG * 64;          // [NW][HG]
    float* ll = mm + NW * HG;                         // [NW][HG]
    float* aa = ll + NW * HG;                         // [HG][R]
    const int pos = pr.tok_pos[t];
    const int* bt = pr.block_table + (int64_t)pr.tok_row[t] * pr.bt_stride;
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    for (int i = threadIdx.x; i < HG * d; i += 64 * NW) {
        const int hh = i / d, c = i % d;
        qs[i] = hh < nh ? q[(int64_t)t * ldq + (int64_t)(h0 + hh) * d + c] : 0.f;
    }
    for (int i = threadIdx.x; i < HG * R; i += 64 * NW) aa[i] = 0.f;
    __syncthreads();
    float m[HG], l[HG], acc[HG][VC];
#pragma unroll
    for (int hh = 0; hh < HG; ++hh) {
        m[hh] = -INFINITY;
        l[hh] = 0.f;
#pragma unroll
        for (int ci = 0; ci < VC; ++ci) acc[hh][ci] = 0.f;
    }
    for (int j0 = lo + 64 * wv; j0 <= pos; j0 += 64 * NW) {
        const int j = j0 + lane;
        float dot[HG];
#pragma unroll
        for (int hh = 0; hh < HG; ++hh) dot[hh] = 0.f;
        if (j <= pos) {
            const int pg = bt[j / pr.page];
            const T_* kr = cache + ((int64_t)pg * pr.page + j % pr.page) * d;
            if (!F32 && (d & 7) == 0) {
                for (int c = 0; c < d; c += 8) {
                    const uint4 kv = ld16(kr + c);
                    const uint32_t w[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float k0 = bf16_lo(w[e]), k1 = bf16_hi(w[e]);
#pragma unroll
                        for (int hh = 0; hh < HG; ++hh) {
                            dot[hh] = fmaf(qs[hh * d + c + 2 * e], k0, dot[hh]);
                            dot[hh] = fmaf(qs[hh * d + c + 2 * e + 1], k1, dot[hh]);
                        }
                    }
                }
            } else {
                for (int c = 0; c < d; ++c) {
                    const float kk = ActL<F32>::ld(kr + c);
#pragma unroll
                    for (int hh = 0; hh < HG; ++hh) dot[hh] = fmaf(qs[hh * d + c], kk, dot[hh]);
                }
            }
        }
        float corr[HG];
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int hh = 0; hh < HG; ++hh) {
            const float s = j <= pos ? dot[hh] * scale : -INFINITY;
            const float mn = fmaxf(m[hh], wave_max(s));
            const float pj = j <= pos ? expf(s - mn) : 0.f;
            corr[hh] = expf(m[hh] - mn);   // m = -inf on the wave's first tile: exp(-inf) = 0
            l[hh] = l[hh] * corr[hh] + wave_sum(pj);
            m[hh] = mn;
            ps[hh * 64 + lane] = pj;
#pragma unroll
            for (int ci = 0; ci < VC; ++ci) acc[hh][ci] *= corr[hh];
        }
        __builtin_amdgcn_wave_barrier();
        const int cnt = pos - j0 + 1 < 64 ? pos - j0 + 1 : 64;
        for (int jj = 0; jj < cnt; jj += 4) {
            const T_* vr[4];
            float pj[HG][4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const bool ok = jj + u < cnt;
                const int jk = ok ? j0 + jj + u : j0;
                const int pg = bt[jk / pr.page];
                vr[u] = cache + ((int64_t)pg * pr.page + jk % pr.page) * d;
#pragma unroll
                for (int hh = 0; hh < HG; ++hh) pj[hh][u] = ok ? ps[hh * 64 + jj + u] : 0.f;
            }
#pragma unroll
            for (int ci = 0; ci < VC; ++ci) {
                const int c = lane + ci * 64;
                if (c < R) {
                    float x[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) x[u] = ActL<F32>::ld(vr[u] + c);
#pragma unroll
                    for (int hh = 0; hh < HG; ++hh)
#pragma unroll
                        for (int u = 0; u < 4; ++u) acc[hh][ci] = fmaf(pj[hh][u], x[u], acc[hh][ci]);
                }
            }
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int hh = 0; hh < HG; ++hh) {
            mm[wv * HG + hh] = m[hh];
            ll[wv * HG + hh] = l[hh];
        }
    }
    __syncthreads();
    // the common maximum (the sink counts as a score), this wave's factor, the denominator
    float fac[HG], L[HG];
#pragma unroll
    for (int hh = 0; hh < HG; ++hh) {
        const float sk = (sinks && hh < nh) ? sinks[h0 + hh] : -INFINITY;
        float M = sk;
        for (int w = 0; w < NW; ++w) M = fmaxf(M, mm[w * HG + hh]);   // wave 0 always has a key: finite
        float tot = sinks ? expf(sk - M) : 0.f;
        for (int w = 0; w < NW; ++w) tot = fmaf(ll[w * HG + hh], expf(mm[w * HG + hh] - M), tot);
        L[hh] = tot;
        fac[hh] = expf(m[hh] - M);
    }
    for (int w = 0; w < NW; ++w) {   // one wave after the other: the order of the sums is fixed
        if (wv == w) {
#pragma unroll
            for (int hh = 0; hh < HG; ++hh)
#pragma unroll
                for (int ci = 0; ci < VC; ++ci) {
                    const int c = lane + ci * 64;
                    if (c < R) aa[hh * R + c] = fmaf(acc[hh][ci], fac[hh], aa[hh * R + c]);
                }
        }
        __syncthreads();
    }
    if (wv == 0) {
#pragma unroll
        for (int hh = 0; hh < HG; ++hh) {
            if (hh >= nh) continue;
#pragma unroll
            for (int ci = 0; ci < VC; ++ci) {
                const int c = lane + ci * 64;
                if (c < R) ActL<F32>::st(out + (int64_t)t * ldo + (int64_t)(h0 + hh) * R + c, aa[hh * R + c] / L[hh]);
            }
        }
    }
}

template <bool F32, int NW, int HG, int VC>
static int launch_latent_attn(const float* q, int64_t ldq, const void* cache, void* out, int64_t ldo, LatentPages pr,
                              const float* sinks, int T, int H, int R, int r, float scale, int window,
                              const int* row_len, int max_len, hipStream_t s) {
    static LdsOptIn done;
    const size_t lds = (size_t)(HG * (R + r) + NW * HG * 64 + 2 * NW * HG + HG * R) * sizeof(float);
    if (lds > 150 * 1024) return MV_ERR_UNSUPPORTED;
    const void* kern = (const void*)latent_attn_kernel<F32, NW, HG, VC>;
    if (lds > 48 * 1024) {
        const int rc = ensure_dynamic_lds(kern, lds, done);
        if (rc != MV_OK) return rc;
    }
    const int groups = (H + HG - 1) / HG;
    hipLaunchKernelGGL((latent_attn_kernel<F32, NW, HG, VC>), dim3((unsigned)((int64_t)T * groups)), dim3(64 * NW), lds, s,
                       q, ldq, cache, out, ldo, pr, sinks, H, R, r, scale, window, row_len, max_len);
    return check_launch();
}

template <bool F32, int NW, int HG>
static int latent_attn_vc(const float* q, int64_t ldq, const void* cache, void* out, int64_t ldo, LatentPages pr,
                          const float* sinks, int T, int H, int R, int r, float scale, int window, const int* row_len,
                          int max_len, hipStream_t s) {
    if (R <= 128) return launch_latent_attn<F32, NW, HG, 2>(q, ldq, cache, out, ldo, pr, sinks, T, H, R, r, scale, window, row_len, max_len, s);
    if (R <= 256) return launch_latent_attn<F32, NW, HG, 4>(q, ldq, cache, out, ldo, pr, sinks, T, H, R, r, scale, window, row_len, max_len, s);
    if (R <= 512) return launch_latent_attn<F32, NW, HG, 8>(q, ldq, cache, out, ldo, pr, sinks, T, H, R, r, scale, window, row_len, max_len, s);
    if (R <= 1024) return launch_latent_attn<F32, NW, HG, 16>(q, ldq, cache, out, ldo, pr, sinks, T, H, R, r, scale, window, row_len, max_len, s);
    return MV_ERR_UNSUPPORTED;
}

// The same attention for a prompt's portion, bf16 pages of 64 tokens: one workgroup per (64 consecutive tokens of a
// row, head), a wave per 16 of them.  A page is staged once in LDS and serves as keys (all R + r columns) and as
// values (the first R).  q . k on v_mfma_f32_16x16x32_bf16 (q rounded to bf16 as the cached latents are), mask,
// sink and softmax in fp32 per lane, P . V on v_mfma_f32_16x16x4_f32 with P staying fp32: a lane's score
// accumulators S[key 16 nt + 4 (lane / 16) + j][query lane % 16] are exactly that instruction's second operand
// for the four keys {16 nt + 4 g + j}, so P never leaves the registers.  KS = (R + r) / 32, CT = R / 16.
typedef __attribute__((ext_vector_type(8))) __bf16 lt_bf16x8_t;

template <int KS, int CT>
__global__ __launch_bounds__(256) void latent_attn_tile_kernel(const float* q, int64_t ldq, const uint16_t* cache,
                                                               uint16_t* out, int64_t ldo, LatentPages pr,
                                                               const int* ch_start, const int* ch_len,
                                                               const float* sinks, int H, float scale, int window) {
    constexpr int D = KS * 32, DV = CT * 16, SK = D + 8;
    extern __shared__ __attribute__((aligned(16))) uint16_t Ks[];   // [64][SK]
    const int ch = blockIdx.x, h = blockIdx.y;
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, r = lane & 15, qd = lane >> 4;
    const int start = ch_start[ch], len = ch_len[ch];
    const int* bt = pr.block_table + (int64_t)pr.tok_row[start] * pr.bt_stride;
    const int p0 = pr.tok_pos[start];            // positions run on from here within the chunk
    const int myq = 16 * wv + r;
    const bool qok = myq < len;
    const int qpos = p0 + myq;
    const int win = window > 0 ? window : (1 << 30);
    lt_bf16x8_t qf[KS];
    {
        const float* qp = q + (int64_t)(start + (qok ? myq : 0)) * ldq + (int64_t)h * D + 8 * qd;
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            const float4 a = *reinterpret_cast<const float4*>(qp + 32 * kk);
            const float4 b = *reinterpret_cast<const float4*>(qp + 32 * kk + 4);
            const uint4 pk = make_uint4(pack_bf16x2(a.x, a.y), pack_bf16x2(a.z, a.w), pack_bf16x2(b.x, b.y),
                                        pack_bf16x2(b.z, b.w));
            qf[kk] = __builtin_bit_cast(lt_bf16x8_t, pk);
        }
    }
    float m = -INFINITY, l = 0.f;
    f32x4_t o[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) o[ct] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const int klo = p0 - win + 1 > 0 ? p0 - win + 1 : 0, khi = p0 + len - 1;
    const int wq_lo = p0 + 16 * wv, wq_hi = wq_lo + 15;   // this wave's query positions
    for (int kt = klo / 64; kt <= khi / 64; ++kt) {
        const int kbase = kt * 64;
        const int64_t pgrow = (int64_t)bt[kt] * 64;
        __syncthreads();
        for (int i = tid; i < 64 * (D / 8); i += 256) {
            const int rr = i / (D / 8), cc = i % (D / 8);
            st16(&Ks[rr * SK + cc * 8], ld16(cache + (pgrow + rr) * D + cc * 8));
        }
        __syncthreads();
        if (kbase > wq_hi || kbase + 63 <= wq_lo - win) continue;   // nothing of this tile is visible to the wave
        f32x4_t sc[4];
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
            sc[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) {
                const lt_bf16x8_t kf = __builtin_bit_cast(lt_bf16x8_t, ld16(&Ks[(16 * nt + r) * SK + 32 * kk + 8 * qd]));
                sc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[kk], sc[nt], 0, 0, 0);
            }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int kpos = kbase + 16 * nt + 4 * qd + j;
                const bool ok = qok && kpos <= qpos && kpos > qpos - win;
                const float v = ok ? sc[nt][j] * scale : -INFINITY;
                sc[nt][j] = v;
                mx = fmaxf(mx, v);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mn = fmaxf(m, mx);
        const float corr = m == -INFINITY ? 0.f : expf(m - mn);
        float ps = 0.f;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float pv = sc[nt][j] == -INFINITY ? 0.f : expf(sc[nt][j] - mn);
                sc[nt][j] = pv;
                ps += pv;
            }
        ps += __shfl_xor(ps, 16, 64);
        ps += __shfl_xor(ps, 32, 64);
        l = l * corr + ps;
        m = mn;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) o[ct] *= corr;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint16_t* vrow = &Ks[(16 * nt + 4 * qd + j) * SK + r];
#pragma unroll
                for (int ct = 0; ct < CT; ++ct)
                    o[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(bf16_bits_to_f32(vrow[16 * ct]), sc[nt][j], o[ct], 0, 0, 0);
            }
    }
    if (qok) {
        // the sink joins the denominator as one more score without a value (a sink far above m: the output goes to zero)
        const float inv = 1.0f / (sinks ? l + expf(sinks[h] - m) : l);
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

template <int KS, int CT>
static int launch_latent_tile(const float* q, int64_t ldq, const void* cache, void* out, int64_t ldo, LatentPages pr,
                              const int* ch_start, const int* ch_len, int chunks, const float* sinks, int H,
                              float scale, int window, hipStream_t s) {
    static LdsOptIn done;
    const size_t lds = (size_t)64 * (KS * 32 + 8) * sizeof(uint16_t);
    const void* kern = (const void*)latent_attn_tile_kernel<KS, CT>;
    if (lds > 48 * 1024) {
        const int rc = ensure_dynamic_lds(kern, lds, done);
        if (rc != MV_OK) return rc;
    }
    hipLaunchKernelGGL((latent_attn_tile_kernel<KS, CT>), dim3(chunks, H), dim3(256), lds, s, q, ldq,
                       (const uint16_t*)cache, (uint16_t*)out, ldo, pr, ch_start, ch_len, sinks, H, scale, window);
    return check_launch();
}

// the (latent width, rotated width) pairs the tile kernel is built for
static bool latent_tile_shape(int R, int r) {
    return (r == 0 || r == 32 || r == 64) && (R == 64 || R == 128 || R == 256 || R == 512) && (R + r) % 32 == 0;
}

}  // namespace mv

extern "C" {

int mv_latent_prep(const float* dkv, int64_t ldkv, const float* w_norm, float eps, void* cache, const float* q,
                   int64_t ldq, void* q_plain, int64_t ldqn, float* q_abs, int64_t ldqa, const double* inv_freq,
                   const int32_t* tok_row, const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int page,
                   int tokens, int heads, int d, int r, int rank, int rot, int interleaved, int f32,
                   mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || heads <= 0 || d <= 0 || r < 0 || rank <= 0 || rot < 0 || rot > r || rot % 2 || page <= 0)
        return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!dkv || !w_norm || !cache || !q || !q_plain || !q_abs || (rot > 0 && !inv_freq) || !tok_row || !tok_pos ||
        !block_table || ldkv < rank + r || ldq < (int64_t)heads * (d + r) || ldqn < (int64_t)heads * d ||
        ldqa < (int64_t)heads * (rank + r))
        return MV_ERR_INVALID_ARG;
    const LatentPages pr{tok_row, tok_pos, block_table, bt_stride, page};
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(latent_prep_kernel<true>, dim3(tokens), dim3(256), 0, s, dkv, ldkv, w_norm, eps, cache, q, ldq, q_plain, ldqn, q_abs, ldqa, inv_freq, pr, heads, d, r, rank, rot, interleaved);
    else hipLaunchKernelGGL(latent_prep_kernel<false>, dim3(tokens), dim3(256), 0, s, dkv, ldkv, w_norm, eps, cache, q, ldq, q_plain, ldqn, q_abs, ldqa, inv_freq, pr, heads, d, r, rank, rot, interleaved);
    return check_launch();
}

int mv_latent_attn(const float* q_abs, int64_t ldq, const void* cache, void* out, int64_t ldo, const int32_t* tok_row,
                   const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int page, const float* sinks,
                   int tokens, int heads, int rank, int r, float scale, int window, int f32, const int32_t* row_len,
                   const int32_t* ch_start, const int32_t* ch_len, int chunks, int max_len, mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || heads <= 0 || rank <= 0 || r < 0 || page <= 0 || window < 0) return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!q_abs || !cache || !out || !tok_row || !tok_pos || !block_table || ldq < (int64_t)heads * (rank + r) ||
        ldo < (int64_t)heads * rank)
        return MV_ERR_INVALID_ARG;
    const LatentPages pr{tok_row, tok_pos, block_table, bt_stride, page};
    hipStream_t s = (hipStream_t)stream;
    // rows of more than max_len tokens (they are cut into the step's chunks) on the matrix cores where the shape fits
    int plain_max = 0;
    if (chunks > 0 && !f32 && page == 64 && heads <= 65535 && latent_tile_shape(rank, r) && row_len && ch_start &&
        ch_len && max_len > 0 && ldq % 4 == 0 && ldo % 4 == 0 && aligned16(q_abs)) {
        int rc = MV_ERR_UNSUPPORTED;
#define MV_LT(R_, r_)                                                                                              \
    if (rank == R_ && r == r_)                                                                                     \
        rc = launch_latent_tile<(R_ + r_) / 32, R_ / 16>(q_abs, ldq, cache, out, ldo, pr, ch_start, ch_len, chunks, \
                                                          sinks, heads, scale, window, s);
        MV_LT(64, 0) MV_LT(128, 0) MV_LT(256, 0) MV_LT(512, 0) MV_LT(64, 32) MV_LT(64, 64) MV_LT(128, 32) MV_LT(128, 64) MV_LT(256, 32) MV_LT(256, 64) MV_LT(512, 32) MV_LT(512, 64)
#undef MV_LT
        if (rc != MV_OK) return rc;
        plain_max = max_len;
    }
    // few tokens (decoding): sixteen waves share a token's keys, so that the launch still fills the chip
    const bool few = (int64_t)tokens * ((heads + 3) / 4) < 2 * (int64_t)num_cus();
    // very few (a handful of decoded tokens): a workgroup per head rather than per four heads
    const bool alone = (int64_t)tokens * ((heads + 3) / 4) < 64;
    if (f32) {
        if (alone) return latent_attn_vc<true, 16, 1>(q_abs, ldq, cache, out, ldo, pr, sinks, tokens, heads, rank, r, scale, window, row_len, plain_max, s);
        if (few) return latent_attn_vc<true, 16, 4>(q_abs, ldq, cache, out, ldo, pr, sinks, tokens, heads, rank, r, scale, window, row_len, plain_max, s);
        return latent_attn_vc<true, 4, 4>(q_abs, ldq, cache, out, ldo, pr, sinks, tokens, heads, rank, r, scale, window, row_len, plain_max, s);
    }
    if (alone) return latent_attn_vc<false, 16, 1>(q_abs, ldq, cache, out, ldo, pr, sinks, tokens, heads, rank, r, scale, window, row_len, plain_max, s);
    if (few) return latent_attn_vc<false, 16, 4>(q_abs, ldq, cache, out, ldo, pr, sinks, tokens, heads, rank, r, scale, window, row_len, plain_max, s);
    return latent_attn_vc<false, 4, 4>(q_abs, ldq, cache, out, ldo, pr, sinks, tokens, heads, rank, r, scale, window, row_len, plain_max, s);
}

}  // extern "C"
