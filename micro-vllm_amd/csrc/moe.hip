// Routed feed-forward (mixture of experts) over a step's tokens, everything on the device so that a step
// can be recorded into a graph:
//
//   moe_route    logits = W_router h in fp32 (h in the activation type), the `top` largest (ties: the lower
//                index), weights = softmax over the chosen logits; beside it sigmoid(w_sg . h), the factor
//                of a shared expert (one number per token)
//   moe_route_scored  scores = softmax of the fp32 logits over ALL router outputs; the `top` largest of
//                score + correction are chosen (ties: the lower index), their weights are the scores themselves
//                (without the correction) divided by their sum (+ floor), times `scale`.  Router outputs from
//                `first_pass` on have no expert behind them: they stand for the input itself (moe_combine)
//   moe_route_sigmoid  the `top` largest fp32 logits (ties: the lower index), weights = sigmoid of each chosen
//                logit, not renormalised
//   gated_act_scaled  rows sorted by expert: out = act( f(s g) * (s u) ) with s the weight of the row's (token,
//                choice) pair - an expert that reads weight * h, formed from the products of h itself (the
//                projections are linear)
//   moe_plan     the step's T * top (token, choice) pairs sorted by expert: seg[e] .. seg[e+1] are expert e's
//                rows, order[i] the pair (token * top + choice) in row i, place[pair] its row.  The order inside
//                an expert is whatever the atomics give; no result depends on it, since a row's products do
//                not depend on the other rows (mv_linear_segments)
//   moe_combine  y_t = sum_k weight[t,k] * expert_out[place[t,k]] (+ factor_t * shared_out_t); with a norm given
//                the sum goes through it straight into the stream: y += tanh(alpha sum) w + b.  A choice
//                ids[t,k] >= first_pass adds weight * pass[t] (the feed-forward's own input) instead of an expert's row
// The experts' products themselves are mv_linear_segments (linear_any.hip) with a SiLU-gate between them.
#include "common.h"

namespace mv {

constexpr int kMaxExperts = 1024, kMaxTop = 16;

template <bool F32>
__global__ __launch_bounds__(256) void moe_route_kernel(const void* h_, int64_t ldh, const float* wr, const float* wsg,
                                                        int* ids, float* wts, float* shared_gate, int n, int E,
                                                        int top, int sigmoid_scores) {
    __shared__ float z[kMaxExperts + 1];
    const int t = blockIdx.x, wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int units = E + (wsg ? 1 : 0);
    for (int e = wv; e < units; e += 4) {
        const float* w = e < E ? wr + (int64_t)e * n : wsg;
        float dot = 0.f;
        if (F32) {
            const float* h = (const float*)h_ + (int64_t)t * ldh;
#pragma unroll 8
            for (int c = lane; c < n; c += 64) dot = fmaf(h[c], w[c], dot);
        } else {
            const uint16_t* h = (const uint16_t*)h_ + (int64_t)t * ldh;
#pragma unroll 8
            for (int c = lane; c < n; c += 64) dot = fmaf(bf16_bits_to_f32(h[c]), w[c], dot);
        }
        dot = wave_sum(dot);
        if (lane == 0) z[e] = dot;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int pick[kMaxTop];
        float val[kMaxTop];
        for (int k = 0; k < top; ++k) {
            int best = -1;
            float bv = -INFINITY;
            for (int e = 0; e < E; ++e) {
                bool taken = false;
                for (int j = 0; j < k; ++j) taken |= pick[j] == e;
                if (!taken && (best < 0 || z[e] > bv)) {
                    best = e;
                    bv = z[e];
                }
            }
            pick[k] = best;
            val[k] = bv;
        }
        float sum = 0.f;
        const float largest = val[0];
        for (int k = 0; k < top; ++k) {
            val[k] = sigmoid_scores ? 1.0f / (1.0f + expf(-val[k])) : expf(val[k] - largest);
            sum += val[k];
        }
        if (sigmoid_scores) sum = 1.0f;      // each chosen expert keeps its own score
        for (int k = 0; k < top; ++k) {
            ids[(int64_t)t * top + k] = pick[k];
            wts[(int64_t)t * top + k] = val[k] / sum;
        }
        if (wsg) shared_gate[t] = 1.0f / (1.0f + expf(-z[E]));
    }
}

template <bool F32>
__global__ __launch_bounds__(256) void moe_route_scored_kernel(const void* h_, int64_t ldh, const float* wr,
                                                               const float* correction, int* ids, float* wts, int n,
                                                               int E, int top, float scale, float floor_) {
    __shared__ float z[kMaxExperts];
    const int t = blockIdx.x, wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int e = wv; e < E; e += 4) {
        const float* w = wr + (int64_t)e * n;
        float dot = 0.f;
        if (F32) {
            const float* h = (const float*)h_ + (int64_t)t * ldh;
#pragma unroll 8
            for (int c = lane; c < n; c += 64) dot = fmaf(h[c], w[c], dot);
        } else {
            const uint16_t* h = (const uint16_t*)h_ + (int64_t)t * ldh;
#pragma unroll 8
            for (int c = lane; c < n; c += 64) dot = fmaf(bf16_bits_to_f32(h[c]), w[c], dot);
        }
        dot = wave_sum(dot);
        if (lane == 0) z[e] = dot;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float largest = z[0], sum = 0.f;
        for (int e = 1; e < E; ++e) largest = fmaxf(largest, z[e]);
        for (int e = 0; e < E; ++e) {
            z[e] = expf(z[e] - largest);
            sum += z[e];
        }
        for (int e = 0; e < E; ++e) z[e] = z[e] / sum;
        int pick[kMaxTop];
        float total = 0.f;
        for (int k = 0; k < top; ++k) {
            int best = -1;
            float bv = -INFINITY;
            for (int e = 0; e < E; ++e) {
                bool taken = false;
                for (int j = 0; j < k; ++j) taken |= pick[j] == e;
                const float c = correction ? z[e] + correction[e] : z[e];
                if (!taken && (best < 0 || c > bv)) {
                    best = e;
                    bv = c;
                }
            }
            pick[k] = best;
            total += z[best];
        }
        total += floor_;
        for (int k = 0; k < top; ++k) {
            ids[(int64_t)t * top + k] = pick[k];
            wts[(int64_t)t * top + k] = (z[pick[k]] / total) * scale;
        }
    }
}

__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* ids, int* seg, int* order, int* place, int pairs,
                                                        int E) {
    __shared__ int cnt[kMaxExperts + 1];
    __shared__ int cur[kMaxExperts];
    for (int e = threadIdx.x; e <= E; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < pairs; i += 1024) atomicAdd(&cnt[ids[i]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int e = 0; e < E; ++e) {
            const int c = cnt[e];
            cur[e] = run;
            seg[e] = run;
            run += c;
        }
        seg[E] = run;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < pairs; i += 1024) {
        const int row = atomicAdd(&cur[ids[i]], 1);
        order[row] = i;
        place[i] = row;
    }
}

// norm_w != NULL: the sum does not go to y but through the norm after the sublayer into the stream,
// x += tanh(alpha sum) w + b, and h (optional) = x in the activation type
template <bool F32>
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* eo, int64_t lde, const int* place,
                                                          const float* wts, const float* so, int64_t lds_,
                                                          const float* shared_gate, float* y, int64_t ldy, int n,
                                                          int top, const float* norm_w, const float* norm_b,
                                                          const float* norm_alpha, void* h_, int64_t ldh,
                                                          const int* ids, int first_pass, const void* pass_,
                                                          int64_t ldp) {
    const int t = blockIdx.x;
    int rows[kMaxTop];
    float w[kMaxTop];
    for (int k = 0; k < top; ++k) {
        rows[k] = place[(int64_t)t * top + k];
        w[k] = wts ? wts[(int64_t)t * top + k] : 1.0f;
        if (ids && ids[(int64_t)t * top + k] >= first_pass) rows[k] = -1;   // the input itself, not an expert's row
    }
    const float g = so ? (shared_gate ? shared_gate[t] : 1.0f) : 0.f;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c < n) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            float v;
            if (rows[k] >= 0) v = eo[(int64_t)rows[k] * lde + c];
            else if (F32) v = ((const float*)pass_)[(int64_t)t * ldp + c];
            else v = bf16_bits_to_f32(((const uint16_t*)pass_)[(int64_t)t * ldp + c]);
            acc = fmaf(w[k], v, acc);
        }
        if (so) acc = fmaf(g, so[(int64_t)t * lds_ + c], acc);
        if (norm_w) {
            acc = y[(int64_t)t * ldy + c] + fmaf(tanhf(norm_alpha[0] * acc), norm_w[c], norm_b[c]);
            if (h_) {
                if (F32) ((float*)h_)[(int64_t)t * ldh + c] = acc;
                else ((uint16_t*)h_)[(int64_t)t * ldh + c] = (uint16_t)f32_to_bf16_bits(acc);
            }
        }
        y[(int64_t)t * ldy + c] = acc;
    }
}

template <bool F32>
__global__ __launch_bounds__(256) void gated_act_scaled_kernel(const float* a, int64_t lda, void* out_, int64_t ldo,
                                                               int n, int kind, float limit, float slope,
                                                               const float* scale, const int* order) {
    const int64_t row = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= n) return;
    const float sc = scale[order ? order[row] : row];
    const float v = gated_act_f(sc * a[row * lda + c], sc * a[row * lda + n + c], kind, limit, slope);
    if (F32) ((float*)out_)[row * ldo + c] = v;
    else ((uint16_t*)out_)[row * ldo + c] = (uint16_t)f32_to_bf16_bits(v);
}

}  // namespace mv

extern "C" {

int mv_moe_route(const void* h, int64_t ldh, const float* w_router, const float* w_shared_gate, int32_t* ids,
                 float* weights, float* shared_gate, int tokens, int n, int experts, int top, int f32,
                 mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || n <= 0 || experts <= 0 || experts > kMaxExperts || top <= 0 || top > kMaxTop || top > experts)
        return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!h || !w_router || !ids || !weights || (w_shared_gate && !shared_gate) || ldh < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(moe_route_kernel<true>, dim3(tokens), dim3(256), 0, s, h, ldh, w_router, w_shared_gate, ids, weights, shared_gate, n, experts, top, 0);
    else hipLaunchKernelGGL(moe_route_kernel<false>, dim3(tokens), dim3(256), 0, s, h, ldh, w_router, w_shared_gate, ids, weights, shared_gate, n, experts, top, 0);
    return check_launch();
}

int mv_moe_route_scored(const void* h, int64_t ldh, const float* w_router, const float* correction, int32_t* ids,
                        float* weights, int tokens, int n, int experts, int top, float scale, float sum_floor, int f32,
                        mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || n <= 0 || experts <= 0 || experts > kMaxExperts || top <= 0 || top > kMaxTop || top > experts)
        return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!h || !w_router || !ids || !weights || ldh < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(moe_route_scored_kernel<true>, dim3(tokens), dim3(256), 0, s, h, ldh, w_router, correction, ids, weights, n, experts, top, scale, sum_floor);
    else hipLaunchKernelGGL(moe_route_scored_kernel<false>, dim3(tokens), dim3(256), 0, s, h, ldh, w_router, correction, ids, weights, n, experts, top, scale, sum_floor);
    return check_launch();
}

int mv_moe_route_sigmoid(const void* h, int64_t ldh, const float* w_router, int32_t* ids, float* weights, int tokens,
                         int n, int experts, int top, int f32, mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || n <= 0 || experts <= 0 || experts > kMaxExperts || top <= 0 || top > kMaxTop || top > experts)
        return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!h || !w_router || !ids || !weights || ldh < n) return MV_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(moe_route_kernel<true>, dim3(tokens), dim3(256), 0, s, h, ldh, w_router, (const float*)nullptr, ids, weights, (float*)nullptr, n, experts, top, 1);
    else hipLaunchKernelGGL(moe_route_kernel<false>, dim3(tokens), dim3(256), 0, s, h, ldh, w_router, (const float*)nullptr, ids, weights, (float*)nullptr, n, experts, top, 1);
    return check_launch();
}

int mv_gated_act_scaled(const float* a, int64_t lda, void* out, int64_t ldo, int rows, int n, int kind, float limit,
                        float slope, const float* scale, const int32_t* order, int f32, mv_stream_t stream) {
    using namespace mv;
    if (rows < 0 || n <= 0 || kind < 0 || kind > 2) return MV_ERR_INVALID_ARG;
    if (rows == 0) return MV_OK;
    if (!a || !out || !scale || lda < 2 * (int64_t)n || ldo < n) return MV_ERR_INVALID_ARG;
    const dim3 grid(rows, (n + 255) / 256);
    hipStream_t s = (hipStream_t)stream;
    if (f32) hipLaunchKernelGGL(gated_act_scaled_kernel<true>, grid, dim3(256), 0, s, a, lda, out, ldo, n, kind, limit, slope, scale, order);
    else hipLaunchKernelGGL(gated_act_scaled_kernel<false>, grid, dim3(256), 0, s, a, lda, out, ldo, n, kind, limit, slope, scale, order);
    return check_launch();
}

int mv_moe_plan(const int32_t* ids, int32_t* seg, int32_t* order, int32_t* place, int pairs, int experts,
                mv_stream_t stream) {
    using namespace mv;
    if (pairs < 0 || experts <= 0 || experts > kMaxExperts) return MV_ERR_INVALID_ARG;
    if (!ids || !seg || !order || !place) return MV_ERR_INVALID_ARG;
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, ids, seg, order, place, pairs,
                       experts);
    return check_launch();
}

int mv_moe_combine(const float* expert_out, int64_t lde, const int32_t* place, const float* weights,
                   const float* shared_out, int64_t lds, const float* shared_gate, float* y, int64_t ldy,
                   const float* norm_w, const float* norm_b, const float* norm_alpha, void* h, int64_t ldh, int tokens,
                   int n, int top, int f32, const int32_t* ids, int first_pass, const void* pass, int64_t ldp,
                   mv_stream_t stream) {
    using namespace mv;
    if (tokens < 0 || n <= 0 || top <= 0 || top > kMaxTop) return MV_ERR_INVALID_ARG;
    if (tokens == 0) return MV_OK;
    if (!expert_out || !place || !y || lde < n || ldy < n ||
        (shared_out && lds < n))
        return MV_ERR_INVALID_ARG;
    if (norm_w ? (!norm_b || !norm_alpha || (h && ldh < n)) : h != nullptr) return MV_ERR_INVALID_ARG;
    if (ids && (!pass || ldp < n || first_pass < 0)) return MV_ERR_INVALID_ARG;
    const dim3 grid(tokens, (n + 255) / 256);
    if (f32) hipLaunchKernelGGL(moe_combine_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream, expert_out, lde, place, weights, shared_out, lds, shared_gate, y, ldy, n, top, norm_w, norm_b, norm_alpha, h, ldh, ids, first_pass, pass, ldp);
    else hipLaunchKernelGGL(moe_combine_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream, expert_out, lde, place, weights, shared_out, lds, shared_gate, y, ldy, n, top, norm_w, norm_b, norm_alpha, h, ldh, ids, first_pass, pass, ldp);
    return check_launch();
}

}  // extern "C"
