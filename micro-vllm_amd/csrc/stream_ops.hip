// Row-wise steps around an fp32 residual stream: layer stacks that keep the running sum of their
// sublayers in 32 bits and hand every projection a copy in the activation type (bf16, or fp32 when
// the whole model runs in 32 bits).
//
//   embed_scaled:        x = table[id] * scale                       (fp32), h = act(x)
//   postnorm_residual:   v = s1*y1 (+ s2*y2); x += v / sqrt(mean(v^2) + eps) * (1 + w); h = act(x)
//                        (the norm sits on the SUBLAYER'S OUTPUT, its weight is stored as an offset
//                        from one)
//   offset_rmsnorm_gather: out = act( x[idx] / sqrt(mean(x[idx]^2) + eps) * (1 + w) )
//   relu_squared:        out = act( max(v, 0)^2 )
//   softcap:             v = cap * tanh(v / cap)
//   dyt_shift:           n = tanh(alpha x) w + b (a norm without statistics); h_t = act( n_t + (n_(t-1) - n_t) mix ),
//                        the last n of every row kept per state slot for the row's next step
//   dyt_gather:          out = act( tanh(alpha x[idx]) w + b )
//   dyt_residual:        x += tanh(alpha y) w + b; h = act(x), or act of the next sublayer's norm of x
//   unitnorm_residual:   x += y / sqrt(mean(y^2) + eps) * w; h = act(x)     (plain weight)
//   rmsnorm_rows:        out = act( v / sqrt(mean(v^2) + eps) * w )         (plain weight, rows of any stride)
//   gelu_gate_rows:      out = act( gelu_tanh(a) * table[id][off .. off+n) )
//   silu_mul:            out = act( silu(a[:, :n]) * a[:, n:2n] )
//   sigmoid_gate:        out = act( a * sigmoid(g) )   (g == NULL: act(a))
//   embed_pair:          x = table[id] * scale + pairs[(prev * mul_prev + id * mul_cur) mod buckets]   (a hashed
//                        table over pairs of neighbouring tokens; row `buckets` where a token has no predecessor);
//                        optionally h = act( x / sqrt(mean(x^2) + eps) * w ), the first layer's norm
//   add_rmsnorm:         x += y1 (+ y2); h = act( x / sqrt(mean(x^2) + eps) * w )   (the sublayers of a parallel
//                        layer enter the stream together and the next layer's norm comes out of the same launch)
//   rmsnorm_gather:      out = act( x[idx] / sqrt(mean(x[idx]^2) + eps) * (offset + w) )
//   gated_act:           out = act( f(a[:, :n]) * a[:, n:2n] ), f = SiLU or the tanh form of GELU; or the clamped
//                        gate  g' = min(g, limit), u' = clamp(u, +-limit): out = act( g' sigmoid(slope g') (u' + 1) )
//   gated_residual_norm: the residual step of a pre-norm layer whose sublayer outputs pass a sigmoid gate:
//                        x += y * sigmoid(g + b)  (mode 1), or  x = y + b  (mode 2: a new pass of a looped span
//                        starts from a projection plus a per-pass vector); then n = x / sqrt(mean(x^2) + eps) *
//                        (offset + w) as fp32 (what a convolution over time reads) and / or in the activation type
//   cast_concat:         out = act( [a | b] )   (two fp32 streams side by side as one projection's operand)
//   gelu_tanh:           out = act( gelu(in) ), the tanh form
//   scale:               v *= s
// All arithmetic is fp32 with the library's exact division, square root and tanh.
#include "common.h"

namespace mv {

template <bool F32> struct Act;
template <> struct Act<true> {
    typedef float T;
    static __device__ __forceinline__ float ld(const float* p) { return *p; }
    static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct Act<false> {
    typedef uint16_t T;
    static __device__ __forceinline__ float ld(const uint16_t* p) { return bf16_bits_to_f32(*p); }
    static __device__ __forceinline__ void st(uint16_t* p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }
};

template <bool F32>
__global__ __launch_bounds__(256) void embed_scaled_kernel(const void* table_, const int* ids, float* x, int64_t ldx,
                                                           void* h_, int64_t ldh, int n, int vocab, float scale) {
    typedef typename Act<F32>::T T;
    const T* table = (const T*)table_;
    T* h = (T*)h_;
    const int row = blockIdx.x;
    int id = ids[row];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    for (int c = threadIdx.x; c < n; c += 256) {
        const float v = Act<F32>::ld(table + (int64_t)id * n + c) * scale;
        x[(int64_t)row * ldx + c] = v;
        Act<F32>::st(h + (int64_t)row * ldh + c, v);
    }
}

template <bool F32>
__global__ __launch_bounds__(256) void postnorm_residual_kernel(const float* y1, int64_t ld1, const float* y2,
                                                                int64_t ld2, float s1, float s2, const float* w,
                                                                float eps, float* x, int64_t ldx, void* h_,
                                                                int64_t ldh, int n) {
    typedef typename Act<F32>::T T;
    __shared__ float red[4];
    T* h = (T*)h_;
    const int row = blockIdx.x;
    const float* a = y1 + (int64_t)row * ld1;
    const float* b = y2 ? y2 + (int64_t)row * ld2 : nullptr;
    float ss = 0.f;
    for (int c = threadIdx.x; c < n; c += 256) {
        const float v = b ? s1 * a[c] + s2 * b[c] : s1 * a[c];
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (int c = threadIdx.x; c < n; c += 256) {
        const float v = b ? s1 * a[c] + s2 * b[c] : s1 * a[c];
        const float s = x[(int64_t)row * ldx + c] + (v * inv) * (1.0f + w[c]);
        x[(int64_t)row * ldx + c] = s;
        Act<F32>::st(h + (int64_t)row * ldh + c, s);
    }
}

template <bool F32>
__global__ __launch_bounds__(256) void offset_rmsnorm_gather_kernel(const float* x, int64_t ldx, const int* idx,
                                                                    const float* w, float eps, float offset,
                                                                    void* out_, int64_t ldo, int n) {
    typedef typename Act<F32>::T T;
    __shared__ float red[4];
    T* out = (T*)out_;
    const int row = blockIdx.x;
    const float* a = x + (int64_t)(idx ? idx[row] : row) * ldx;
    float ss = 0.f;
    for (int c = threadIdx.x; c < n; c += 256) ss += a[c] * a[c];
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (int c = threadIdx.x; c < n; c += 256) Act<F32>::st(out + (int64_t)row * ldo + c, (a[c] * inv) * (offset + w[c]));
}

template <bool F32>
__global__ __launch_bounds__(256) void relu_squared_kernel(const float* in, int64_t ldi, void* out_, int64_t ldo,
                                                           int n) {
    typedef typename Act<F32>::T T;
    T* out = (T*)out_;
    const int row = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= n) return;
    const float v = fmaxf(in[(int64_t)row * ldi + c], 0.f);
    Act<F32>::st(out + (int64_t)row * ldo + c, v * v);
}

__global__ __launch_bounds__(256) void softcap_kernel(float* v, int64_t count, float cap) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count) v[i] = cap * tanhf(v[i] / cap);
}

// ---- Dynamic Tanh norm, token shift ------------------------------------------------------------------
// One workgroup per token.  n_(t-1) of a row's first token is the slot's kept vector (zeros when the
// sequence holds nothing yet); the workgroup of that first token also writes the row's LAST n into the
// slot, so that nobody else touches the slot in this launch.
template <bool F32>
__global__ __launch_bounds__(256) void dyt_shift_kernel(const float* x, int64_t ldx, const float* w, const float* b,
                                                        const float* alpha, const float* mix, float* state,
                                                        void* h_, int64_t ldh, const int* tok_row,
                                                        const int* row_start, const int* row_len, const int* row_ctx,
                                                        const int* row_slot, int n) {
    typedef typename Act<F32>::T T;
    T* h = (T*)h_;
    const int t = blockIdx.x, r = tok_row[t];
    const int first = row_start[r], len = row_len[r];
    const float al = alpha[0];
    const float* cur = x + (int64_t)t * ldx;
    const bool head = t == first;
    float* kept = state + (int64_t)row_slot[r] * n;
    const bool carried = row_ctx[r] > 0;
    const float* prev = x + (int64_t)(t - 1) * ldx;
    const float* last = x + (int64_t)(first + len - 1) * ldx;
    // one value per thread (blockIdx.y walks the row): a row alone in its step is spread over many workgroups
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c < n) {
        const float nc = fmaf(tanhf(al * cur[c]), w[c], b[c]);
        float np;
        if (head) np = carried ? kept[c] : 0.f;
        else np = fmaf(tanhf(al * prev[c]), w[c], b[c]);
        Act<F32>::st(h + (int64_t)t * ldh + c, fmaf(np - nc, mix[c], nc));
        if (head) kept[c] = len == 1 ? nc : fmaf(tanhf(al * last[c]), w[c], b[c]);
    }
}

template <bool F32>
__global__ __launch_bounds__(256) void dyt_gather_kernel(const float* x, int64_t ldx, const int* idx, const float* w,
                                                         const float* b, const float* alpha, void* out_, int64_t ldo,
                                                         int n) {
    typedef typename Act<F32>::T T;
    T* out = (T*)out_;
    const int row = blockIdx.x;
    const float* a = x + (int64_t)(idx ? idx[row] : row) * ldx;
    const float al = alpha[0];
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c < n) Act<F32>::st(out + (int64_t)row * ldo + c, fmaf(tanhf(al * a[c]), w[c], b[c]));
}

// w2 != NULL: h receives the NEXT sublayer's norm of the new x, tanh(alpha2 x) w2 + b2, instead of x itself
template <bool F32>
__global__ __launch_bounds__(256) void dyt_residual_kernel(const float* y, int64_t ldy, const float* w, const float* b,
                                                           const float* alpha, float* x, int64_t ldx, void* h_,
                                                           int64_t ldh, int n, const float* w2, const float* b2,
                                                           const float* alpha2) {
    typedef typename Act<F32>::T T;
    T* h = (T*)h_;
    const int row = blockIdx.x;
    const float al = alpha[0];
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c < n) {
        const float s = x[(int64_t)row * ldx + c] + fmaf(tanhf(al * y[(int64_t)row * ldy + c]), w[c], b[c]);
        x[(int64_t)row * ldx + c] = s;
        if (h) Act<F32>::st(h + (int64_t)row * ldh + c, w2 ? fmaf(tanhf(alpha2[0] * s), w2[c], b2[c]) : s);
    }
}

template <bool F32>
__global__ __launch_bounds__(256) void unitnorm_residual_kernel(const float* y, int64_t ldy, const float* w, float eps,
                                                                float* x, int64_t ldx, void* h_, int64_t ldh, int n) {
    typedef typename Act<F32>::T T;
    __shared__ float red[4];
    T* h = (T*)h_;
    const int row = blockIdx.x;
    const float* a = y + (int64_t)row * ldy;
    float ss = 0.f;
#pragma unroll 4
    for (int c = threadIdx.x; c < n; c += 256) ss += a[c] * a[c];
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
#pragma unroll 4
    for (int c = threadIdx.x; c < n; c += 256) {
        const float s = x[(int64_t)row * ldx + c] + (a[c] * inv) * w[c];
        x[(int64_t)row * ldx + c] = s;
        if (h) Act<F32>::st(h + (int64_t)row * ldh + c, s);
    }
}

// one wave per row of `n` values (rows may be heads of a wider buffer: row r starts at (r / per) * ld + (r % per) * n)
template <bool F32>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const float* v, int64_t ld, int per, const float* w,
                                                           float eps, void* out_, int64_t ldo, int64_t rows, int n) {
    typedef typename Act<F32>::T T;
    T* out = (T*)out_;
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (r >= rows) return;
    const float* a = v + (r / per) * ld + (r % per) * n;
    T* o = out + (r / per) * ldo + (r % per) * n;
    float ss = 0.f;
#pragma unroll 4
    for (int c = lane; c < n; c += 64) ss += a[c] * a[c];
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
#pragma unroll 4
    for (int c = lane; c < n; c += 64) Act<F32>::st(o + c, (a[c] * inv) * w[c]);
}

template <bool F32>
__global__ __launch_bounds__(256) void gelu_gate_rows_kernel(const float* a, int64_t lda, const void* table_,
                                                             int64_t ldt, int off, const int* ids, int vocab,
                                                             void* out_, int64_t ldo, int n) {
    typedef typename Act<F32>::T T;
    const T* table = (const T*)table_;
    T* out = (T*)out_;
    const int row = blockIdx.x;
    int id = ids[row];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c < n) {
        const float e = Act<F32>::ld(table + (int64_t)id * ldt + off + c);
        Act<F32>::st(out + (int64_t)row * ldo + c, gelu_tanh_f(a[(int64_t)row * lda + c]) * e);
    }
}

template <bool F32>
__global__ __launch_bounds__(256) void silu_mul_kernel(const float* a, int64_t lda, void* out_, int64_t ldo, int n) {
    typedef typename Act<F32>::T T;
    T* out = (T*)out_;
    const int64_t row = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= n) return;
    const float g = a[row * lda + c], u = a[row * lda + n + c];
    Act<F32>::st(out + row * ldo + c, (g / (1.0f + expf(-g))) * u);
}

template <bool F32>
__global__ __launch_bounds__(256) void sigmoid_gate_kernel(const float* a, int64_t lda, const float* g, int64_t ldg,
                                                           void* out_, int64_t ldo, int n) {
    typedef typename Act<F32>::T T;
    T* out = (T*)out_;
    const int64_t row = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= n) return;
    float v = a[row * lda + c];
    if (g) v = v / (1.0f + expf(-g[row * ldg + c]));
    Act<F32>::st(out + row * ldo + c, v);
}

// ---- pair-hashed embedding, parallel layers behind one norm, gated activations ----------------------------
template <bool F32>
__global__ __launch_bounds__(256) void embed_pair_kernel(const void* table_, const void* pairs_, const int* ids,
                                                         const int* prev, float* x, int64_t ldx, int n, int vocab,
                                                         int64_t buckets, int64_t mul_prev, int64_t mul_cur,
                                                         float scale, const float* norm_w, float eps, void* h_,
                                                         int64_t ldh) {
    typedef typename Act<F32>::T T;
    __shared__ float red[4];
    const T* table = (const T*)table_;
    const T* pairs = (const T*)pairs_;
    const int row = blockIdx.x;
    int id = ids[row];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const int pv = prev[row];
    // every factor reduced first: the products stay below 2^62 for any 31-bit bucket count
    const int64_t r = pv < 0 ? buckets
                             : (((int64_t)pv % buckets) * (mul_prev % buckets) % buckets +
                                ((int64_t)id % buckets) * (mul_cur % buckets) % buckets) % buckets;
    float ss = 0.f;
    for (int c = threadIdx.x; c < n; c += 256) {
        const float v = Act<F32>::ld(table + (int64_t)id * n + c) * scale + Act<F32>::ld(pairs + r * n + c);
        x[(int64_t)row * ldx + c] = v;
        ss += v * v;
    }
    if (!norm_w) return;
    // the first layer's norm of the row out of the same launch
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (int c = threadIdx.x; c < n; c += 256)
        Act<F32>::st((T*)h_ + (int64_t)row * ldh + c, (x[(int64_t)row * ldx + c] * inv) * norm_w[c]);
}

template <bool F32>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(const float* y1, int64_t ld1, const float* y2, int64_t ld2,
                                                          float* x, int64_t ldx, const float* w, float eps, void* h_,
                                                          int64_t ldh, int n) {
    typedef typename Act<F32>::T T;
    __shared__ float red[4];
    T* h = (T*)h_;
    const int row = blockIdx.x;
    float* xr = x + (int64_t)row * ldx;
    float ss = 0.f;
#pragma unroll 4
    for (int c = threadIdx.x; c < n; c += 256) {
        float v = xr[c];
        if (y1) {
            v += y2 ? y1[(int64_t)row * ld1 + c] + y2[(int64_t)row * ld2 + c] : y1[(int64_t)row * ld1 + c];
            xr[c] = v;
        }
        ss += v * v;
    }
    if (!w) return;
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
#pragma unroll 4
    for (int c = threadIdx.x; c < n; c += 256) Act<F32>::st(h + (int64_t)row * ldh + c, (xr[c] * inv) * w[c]);
}

template <bool F32>
__global__ __launch_bounds__(256) void gated_act_kernel(const float* a, int64_t lda, void* out_, int64_t ldo, int n,
                                                        int kind, float limit, float slope) {
    typedef typename Act<F32>::T T;
    T* out = (T*)out_;
    const int64_t row = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= n) return;
    Act<F32>::st(out + row * ldo + c, gated_act_f(a[row * lda + c], a[row * lda + n + c], kind, limit, slope));
}


// mode 0: x as it is; 1: x += y * sigmoid(g + b); 2: x = y + b.  w != NULL: the norm of the new x, to n32 (fp32)
// and / or h (activation type)
template <bool F32>
__global__ __launch_bounds__(256) void gated_residual_norm_kernel(const float* y, int64_t ldy, const float* g,
                                                                  int64_t ldg, const float* b, int mode, float* x,
                                                                  int64_t ldx, const float* w, float eps, float offset,
                                                                  float* n32, int64_t ldn, void* h_, int64_t ldh,
                                                                  int n) {
    typedef typename Act<F32>::T T;
    __shared__ float red[4];
    T* h = (T*)h_;
    const int64_t row = blockIdx.x;
    float* xr = x + row * ldx;
    float ss = 0.f;
#pragma unroll 4
    for (int c = threadIdx.x; c < n; c += 256) {
        float v;
        if (mode == 1) {
            const float z = g[row * ldg + c] + (b ? b[c] : 0.f);
            v = fmaf(y[row * ldy + c], 1.0f / (1.0f + expf(-z)), xr[c]);
            xr[c] = v;
        } else if (mode == 2) {
            v = y[row * ldy + c] + (b ? b[c] : 0.f);
            xr[c] = v;
        } else {
            v = xr[c];
        }
        ss += v * v;
    }
    if (!w) return;
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
#pragma unroll 4
    for (int c = threadIdx.x; c < n; c += 256) {
        const float v = (xr[c] * inv) * (offset + w[c]);
        if (n32) n32[row * ldn + c] = v;
        if (h) Act<F32>::st(h + row * ldh + c, v);
    }
}

template <bool F32>
__global__ __launch_bounds__(256) void cast_concat_kernel(const float* a, int64_t lda, const float* b, int64_t ldb,
                                                          void* out_, int64_t ldo, int n) {
    typedef typename Act<F32>::T T;
    T* out = (T*)out_;
    const int64_t row = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= 2 * n) return;
    Act<F32>::st(out + row * ldo + c, c < n ? a[row * lda + c] : b[row * ldb + (c - n)]);
}

template <bool F32>
__global__ __launch_bounds__(256) void gelu_tanh_kernel(const float* in, int64_t ldi, void* out_, int64_t ldo, int n) {
    typedef typename Act<F32>::T T;
    T* out = (T*)out_;
    const int64_t row = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c < n) Act<F32>::st(out + row * ldo + c, gelu_tanh_f(in[row * ldi + c]));
}

__global__ __launch_bounds__(256) void scale_kernel(float* v, int64_t count, float s) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count) v[i] *= s;
}

}  // namespace mv

extern "C" {

int mv_embed_scaled(const void* table, const int32_t* ids, float* x, int64_t ldx, void* h, int64_t ldh, int rows,
                    int n, int vocab, float scale, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0 || vocab <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!table || !ids || !x || !h || ldx < n || ldh < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(embed_scaled_kernel<true>, dim3(rows), dim3(256), 0, s, table, ids, x, ldx, h, ldh, n, vocab, scale);
    else hipLaunchKernelGGL(embed_scaled_kernel<false>, dim3(rows), dim3(256), 0, s, table, ids, x, ldx, h, ldh, n, vocab, scale);
    return check_launch();
}

int mv_postnorm_residual(const float* y1, int64_t ld1, const float* y2, int64_t ld2, float s1, float s2,
                         const float* w, float eps, float* x, int64_t ldx, void* h, int64_t ldh, int rows, int n,
                         int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!y1 || !w || !x || !h || ld1 < n || (y2 && ld2 < n) || ldx < n || ldh < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(postnorm_residual_kernel<true>, dim3(rows), dim3(256), 0, s, y1, ld1, y2, ld2, s1, s2, w, eps, x, ldx, h, ldh, n);
    else hipLaunchKernelGGL(postnorm_residual_kernel<false>, dim3(rows), dim3(256), 0, s, y1, ld1, y2, ld2, s1, s2, w, eps, x, ldx, h, ldh, n);
    return check_launch();
}

int mv_offset_rmsnorm_gather(const float* x, int64_t ldx, const int32_t* idx, const float* w, float eps, void* out,
                             int64_t ldo, int rows, int n, int f32, mv_stream_t stream) {
    return mv_rmsnorm_gather(x, ldx, idx, w, eps, 1.0f, out, ldo, rows, n, f32, stream);
}

int mv_rmsnorm_gather(const float* x, int64_t ldx, const int32_t* idx, const float* w, float eps, float offset,
                      void* out, int64_t ldo, int rows, int n, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!x || !w || !out || ldx < n || ldo < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(offset_rmsnorm_gather_kernel<true>, dim3(rows), dim3(256), 0, s, x, ldx, idx, w, eps, offset, out, ldo, n);
    else hipLaunchKernelGGL(offset_rmsnorm_gather_kernel<false>, dim3(rows), dim3(256), 0, s, x, ldx, idx, w, eps, offset, out, ldo, n);
    return check_launch();
}

int mv_embed_pair(const void* table, const void* pairs, const int32_t* ids, const int32_t* prev, float* x, int64_t ldx,
                  int rows, int n, int vocab, int64_t buckets, int64_t mul_prev, int64_t mul_cur, float scale,
                  const float* norm_w, float eps, void* h, int64_t ldh, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0 || vocab <= 0 || buckets <= 0 || buckets > 0x7fffffff || mul_prev < 0 || mul_cur < 0)
        return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!table || !pairs || !ids || !prev || !x || ldx < n || (norm_w && (!h || ldh < n))) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(embed_pair_kernel<true>, dim3(rows), dim3(256), 0, s, table, pairs, ids, prev, x, ldx, n, vocab, buckets, mul_prev, mul_cur, scale, norm_w, eps, h, ldh);
    else hipLaunchKernelGGL(embed_pair_kernel<false>, dim3(rows), dim3(256), 0, s, table, pairs, ids, prev, x, ldx, n, vocab, buckets, mul_prev, mul_cur, scale, norm_w, eps, h, ldh);
    return check_launch();
}

int mv_add_rmsnorm(const float* y1, int64_t ld1, const float* y2, int64_t ld2, float* x, int64_t ldx, const float* w,
                   float eps, void* h, int64_t ldh, int rows, int n, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!x || ldx < n || (y1 && ld1 < n) || (y2 && (!y1 || ld2 < n)) || (w && (!h || ldh < n)) || (!w && !y1))
        return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(add_rmsnorm_kernel<true>, dim3(rows), dim3(256), 0, s, y1, ld1, y2, ld2, x, ldx, w, eps, h, ldh, n);
    else hipLaunchKernelGGL(add_rmsnorm_kernel<false>, dim3(rows), dim3(256), 0, s, y1, ld1, y2, ld2, x, ldx, w, eps, h, ldh, n);
    return check_launch();
}

int mv_gated_act(const float* a, int64_t lda, void* out, int64_t ldo, int rows, int n, int kind, float limit,
                 float slope, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0 || kind < 0 || kind > 2) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!a || !out || lda < 2 * (int64_t)n || ldo < n) return MV_ERR_INVALID_ARG;
    const dim3 grid(rows, (n + 255) / 256);
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(gated_act_kernel<true>, grid, dim3(256), 0, s, a, lda, out, ldo, n, kind, limit, slope);
    else hipLaunchKernelGGL(gated_act_kernel<false>, grid, dim3(256), 0, s, a, lda, out, ldo, n, kind, limit, slope);
    return check_launch();
}

int mv_relu_squared(const float* in, int64_t ldi, void* out, int64_t ldo, int rows, int n, int f32,
                    mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!in || !out || ldi < n || ldo < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(rows, (n + 255) / 256);
    if (f32) hipLaunchKernelGGL(relu_squared_kernel<true>, grid, dim3(256), 0, s, in, ldi, out, ldo, n);
    else hipLaunchKernelGGL(relu_squared_kernel<false>, grid, dim3(256), 0, s, in, ldi, out, ldo, n);
    return check_launch();
}

int mv_softcap(float* v, int64_t count, float cap, mv_stream_t stream) {
    using namespace mv;
    if (count < 0 || !(cap > 0.f)) return MV_ERR_INVALID_ARG;
    if (count == 0) return MV_OK;
    if (!v) return MV_ERR_INVALID_ARG;
    hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, (hipStream_t)stream, v, count, cap);
    return check_launch();
}

#define MV_F32_LAUNCH(kern, grid, ...)                                                              \
    do {                                                                                            \
        if (f32) hipLaunchKernelGGL(kern<true>, grid, dim3(256), 0, s, __VA_ARGS__);                \
        else hipLaunchKernelGGL(kern<false>, grid, dim3(256), 0, s, __VA_ARGS__);                   \
    } while (0)

int mv_dyt_shift(const float* x, int64_t ldx, const float* w, const float* b, const float* alpha, const float* mix,
                 float* state, void* h, int64_t ldh, const int32_t* tok_row, const int32_t* row_start,
                 const int32_t* row_len, const int32_t* row_ctx, const int32_t* row_slot, int tokens, int n, int f32,
                 mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!x || !w || !b || !alpha || !mix || !state || !h || !tok_row || !row_start || !row_len || !row_ctx ||
        !row_slot || ldx < n || ldh < n)
        return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    MV_F32_LAUNCH(dyt_shift_kernel, dim3(tokens, (n + 255) / 256), x, ldx, w, b, alpha, mix, state, h, ldh, tok_row, row_start, row_len,
                  row_ctx, row_slot, n);
    return check_launch();
}

int mv_dyt_gather(const float* x, int64_t ldx, const int32_t* idx, const float* w, const float* b, const float* alpha,
                  void* out, int64_t ldo, int rows, int n, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!x || !w || !b || !alpha || !out || ldx < n || ldo < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    MV_F32_LAUNCH(dyt_gather_kernel, dim3(rows, (n + 255) / 256), x, ldx, idx, w, b, alpha, out, ldo, n);
    return check_launch();
}

int mv_dyt_residual(const float* y, int64_t ldy, const float* w, const float* b, const float* alpha, float* x,
                    int64_t ldx, void* h, int64_t ldh, const float* w2, const float* b2, const float* alpha2, int rows,
                    int n, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!y || !w || !b || !alpha || !x || ldy < n || ldx < n || (h && ldh < n)) return MV_ERR_INVALID_ARG;
    if (w2 && (!b2 || !alpha2 || !h)) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    MV_F32_LAUNCH(dyt_residual_kernel, dim3(rows, (n + 255) / 256), y, ldy, w, b, alpha, x, ldx, h, ldh, n, w2, b2, alpha2);
    return check_launch();
}

int mv_unitnorm_residual(const float* y, int64_t ldy, const float* w, float eps, float* x, int64_t ldx, void* h,
                         int64_t ldh, int rows, int n, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!y || !w || !x || ldy < n || ldx < n || (h && ldh < n)) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    MV_F32_LAUNCH(unitnorm_residual_kernel, dim3(rows), y, ldy, w, eps, x, ldx, h, ldh, n);
    return check_launch();
}

int mv_rmsnorm_rows(const float* v, int64_t ld, int per, const float* w, float eps, void* out, int64_t ldo,
                    int rows, int n, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0 || per <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!v || !w || !out || ld < (int64_t)per * n || ldo < (int64_t)per * n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    const int64_t total = (int64_t)rows * per;
    MV_F32_LAUNCH(rmsnorm_rows_kernel, dim3((unsigned)((total + 3) / 4)), v, ld, per, w, eps, out, ldo, total, n);
    return check_launch();
}

int mv_gelu_gate_rows(const float* a, int64_t lda, const void* table, int64_t ldt, int off, const int32_t* ids,
                      int vocab, void* out, int64_t ldo, int rows, int n, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0 || vocab <= 0 || off < 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!a || !table || !ids || !out || lda < n || ldt < off + n || ldo < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    MV_F32_LAUNCH(gelu_gate_rows_kernel, dim3(rows, (n + 255) / 256), a, lda, table, ldt, off, ids, vocab, out, ldo, n);
    return check_launch();
}

int mv_silu_mul(const float* a, int64_t lda, void* out, int64_t ldo, int rows, int n, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!a || !out || lda < 2 * (int64_t)n || ldo < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(rows, (n + 255) / 256);
    MV_F32_LAUNCH(silu_mul_kernel, grid, a, lda, out, ldo, n);
    return check_launch();
}

int mv_sigmoid_gate(const float* a, int64_t lda, const float* g, int64_t ldg, void* out, int64_t ldo, int rows, int n,
                    int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!a || !out || lda < n || (g && ldg < n) || ldo < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(rows, (n + 255) / 256);
    MV_F32_LAUNCH(sigmoid_gate_kernel, grid, a, lda, g, ldg, out, ldo, n);
    return check_launch();
}

int mv_gated_residual_norm(const float* y, int64_t ldy, const float* g, int64_t ldg, const float* b, int mode, float* x,
                           int64_t ldx, const float* w, float eps, float offset, float* n32, int64_t ldn, void* h,
                           int64_t ldh, int rows, int n, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0 || mode < 0 || mode > 2) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!x || ldx < n || (mode != 0 && (!y || ldy < n)) || (mode == 1 && (!g || ldg < n)) ||
        (w && !n32 && !h) || (!w && (n32 || h)) || (n32 && ldn < n) || (h && ldh < n) || (!w && mode == 0))
        return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(gated_residual_norm_kernel<true>, dim3(rows), dim3(256), 0, s, y, ldy, g, ldg, b, mode, x, ldx, w, eps, offset, n32, ldn, h, ldh, n);
    else hipLaunchKernelGGL(gated_residual_norm_kernel<false>, dim3(rows), dim3(256), 0, s, y, ldy, g, ldg, b, mode, x, ldx, w, eps, offset, n32, ldn, h, ldh, n);
    return check_launch();
}

int mv_cast_concat(const float* a, int64_t lda, const float* b, int64_t ldb, void* out, int64_t ldo, int rows, int n,
                   int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!a || !b || !out || lda < n || ldb < n || ldo < 2 * (int64_t)n) return MV_ERR_INVALID_ARG;
    const dim3 grid(rows, (2 * n + 255) / 256);
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(cast_concat_kernel<true>, grid, dim3(256), 0, s, a, lda, b, ldb, out, ldo, n);
    else hipLaunchKernelGGL(cast_concat_kernel<false>, grid, dim3(256), 0, s, a, lda, b, ldb, out, ldo, n);
    return check_launch();
}

int mv_gelu_tanh(const float* in, int64_t ldi, void* out, int64_t ldo, int rows, int n, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!in || !out || ldi < n || ldo < n) return MV_ERR_INVALID_ARG;
    const dim3 grid(rows, (n + 255) / 256);
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(gelu_tanh_kernel<true>, grid, dim3(256), 0, s, in, ldi, out, ldo, n);
    else hipLaunchKernelGGL(gelu_tanh_kernel<false>, grid, dim3(256), 0, s, in, ldi, out, ldo, n);
    return check_launch();
}

int mv_scale(float* v, int64_t count, float factor, mv_stream_t stream) {
    using namespace mv;
    if (count < 0) return MV_ERR_INVALID_ARG;
    if (count == 0) return MV_OK;
    if (!v) return MV_ERR_INVALID_ARG;
    hipLaunchKernelGGL(scale_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, (hipStream_t)stream, v, count,
                       factor);
    return check_launch();
}

}  // extern "C"
