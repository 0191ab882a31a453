// A feed-forward made of many small gated feed-forwards ("experts"), of which every row uses a few, chosen by a router.
//
//   gi_route_top         the router's choice per row: scores (sigmoid of the logits, or a softmax over them), the `top` largest
//                        (the lower index wins a tie), optionally divided by their sum
//   gi_experts_gate_up   mid[(row, choice)] = act(W_gate[e] a) * (W_up[e] a), e the row's choice and a the row, multiplied by the
//                        choice's score first where the score weighs the expert's input
//   gi_experts_down      x[row] (+)= sum over the row's choices of (score, where it weighs the output) * W_down[e] mid[(row, choice)]
//
// These two walk the weights of each (row, choice) with one wave per output: the form for the few rows of decoding steps, where
// every row reads its own experts and the weights' bytes are the cost.  Every sum is a lane's own share in a fixed order, then the
// lanes by a butterfly, then the choices one after the other: nothing depends on the batch.
#include "common.h"

namespace {

__device__ __forceinline__ float act_of(float z, int act) {
    return act == 1 ? 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))) : z / (1.0f + expf(-z));
}

constexpr int ROUTE_PER_LANE = 16;      // experts a lane looks at: up to 1024 experts

// One wave per row.  score_kind 0: sigmoid, 1: softmax over all experts.
__global__ __launch_bounds__(64) void route_top_kernel(const float* __restrict__ logits, long ld, int n_experts, int top, int score_kind, int renormalize,
                                                      int* __restrict__ ids, float* __restrict__ weights) {
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x;
    float z[ROUTE_PER_LANE];
    float biggest = -INFINITY;
#pragma unroll
    for (int i = 0; i < ROUTE_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        z[i] = e < n_experts ? logits[t * ld + e] : -INFINITY;
        biggest = fmaxf(biggest, z[i]);
    }
    float denominator = 1.0f;
    if (score_kind == 1) {
        biggest = wave_max(biggest);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < ROUTE_PER_LANE; ++i) s += lane + 64 * i < n_experts ? expf(z[i] - biggest) : 0.f;
        denominator = wave_sum(s);
    }
    float total = 0.f, mine = 0.f;
    int my_id = 0;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < ROUTE_PER_LANE; ++i) {
            if (z[i] > best) best = z[i], at = lane + 64 * i;          // (ascending index within the lane: the first of equals stays)
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, 64);
            const int oa = __shfl_xor(at, off, 64);
            if (ob > best || (ob == best && oa < at)) best = ob, at = oa;
        }
        const float score = score_kind == 1 ? expf(best - biggest) / denominator : 1.0f / (1.0f + expf(-best));
        total += score;
        if (lane == k) mine = score, my_id = at;
#pragma unroll
        for (int i = 0; i < ROUTE_PER_LANE; ++i) {
            if (lane + 64 * i == at) z[i] = -INFINITY;
        }
    }
    if (lane < top) {
        ids[t * top + lane] = my_id;
        weights[t * top + lane] = renormalize ? mine / total : mine;
    }
}

// One wave per (row, choice, output j): both dot products over the row, the lanes' shares of k interleaved.
template <typename TW, typename TA, typename TO>
__global__ __launch_bounds__(256) void experts_gate_up_kernel(const TA* __restrict__ h, long ldh, const TW* __restrict__ w_gate, const TW* __restrict__ w_up,
                                                             const int* __restrict__ ids, const float* __restrict__ weights, int weigh_input,
                                                             int top, TO* __restrict__ mid, long ldm, int width, int ff, int act) {
    const size_t item = blockIdx.x;                     // (row * top + choice)
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int j = blockIdx.y * 4 + wave;
    if (j >= ff) return;
    const size_t row = item / top, e = ids[item];
    const float s = weigh_input ? weights[item] : 1.0f;
    const TA* a = h + row * ldh;
    const TW* g = w_gate + (e * ff + j) * (size_t)width;
    const TW* u = w_up + (e * ff + j) * (size_t)width;
    float sg = 0.f, su = 0.f;
    for (int d = lane; d < width; d += 64) {
        float v = s * load_f32(a, d);
        if (sizeof(TA) == 2) v = bf16_to_f32(f32_to_bf16(v));      // rows that go into a product are stored as the product reads them
        sg = fmaf(load_f32(g, d), v, sg);
        su = fmaf(load_f32(u, d), v, su);
    }
    sg = wave_sum(sg);
    su = wave_sum(su);
    if (lane == 0) store_f32(mid + item * ldm, j, act_of(sg, act) * su);
}

template <typename TW, typename TM>
__global__ __launch_bounds__(256) void experts_down_kernel(const TM* __restrict__ mid, long ldm, const TW* __restrict__ w_down, const int* __restrict__ ids,
                                                          const float* __restrict__ weights, int weigh_output, int top, float* __restrict__ x, long ldx,
                                                          int width, int ff, int accumulate) {
    const size_t row = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = blockIdx.y * 4 + wave;
    if (c >= width) return;
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
        const size_t item = row * top + k, e = ids[item];
        const TM* m = mid + item * ldm;
        const TW* w = w_down + (e * width + c) * (size_t)ff;
        float s = 0.f;
        for (int d = lane; d < ff; d += 64) s = fmaf(load_f32(w, d), load_f32(m, d), s);
        s = wave_sum(s);
        total += weigh_output ? weights[item] * s : s;
    }
    if (lane == 0) x[row * ldx + c] = accumulate ? x[row * ldx + c] + total : total;
}

}  // namespace

GI_API int gi_route_top(const float* logits, long ld, int n_rows, int n_experts, int top, int score_kind, int renormalize, int* ids, float* weights, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_experts > 0 && n_experts <= 64 * ROUTE_PER_LANE && top > 0 && top <= n_experts && top <= 64 && ld >= n_experts && (score_kind == 0 || score_kind == 1),
               "route_top: bad sizes (rows %d, experts %d, top %d)", n_rows, n_experts, top);
    route_top_kernel<<<n_rows, 64, 0, stream>>>(logits, ld, n_experts, top, score_kind, renormalize, ids, weights);
    GI_CHECK_LAUNCH("route_top");
    return 0;
}

GI_API int gi_experts_gate_up(const void* h, int h_dtype, long ldh, const void* w_gate, const void* w_up, int w_dtype, const int* ids, const float* weights,
                              int weigh_input, void* mid, int mid_dtype, long ldm, int n_rows, int top, int width, int ff, int act, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && top > 0 && top <= 65535 && width > 0 && ff > 0 && ldh >= width && ldm >= ff && (act == 0 || act == 1) && (long)n_rows * top < (1l << 31),
               "experts_gate_up: bad sizes (rows %d, top %d, width %d, ff %d)", n_rows, top, width, ff);
    dim3 grid(n_rows * top, (ff + 3) / 4);
    GI_REQUIRE(grid.y <= 65535, "experts_gate_up: experts too wide");
#define LAUNCH(TW, TA, TO)                                                                                                                      \
    experts_gate_up_kernel<TW, TA, TO><<<grid, 256, 0, stream>>>((const TA*)h, ldh, (const TW*)w_gate, (const TW*)w_up, ids, weights, weigh_input, \
                                                                 top, (TO*)mid, ldm, width, ff, act)
    if (w_dtype == GI_BF16 && h_dtype == GI_BF16 && mid_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t, bf16_t);
    else if (w_dtype == GI_F32 && h_dtype == GI_F32 && mid_dtype == GI_F32) LAUNCH(float, float, float);
    else if (w_dtype == GI_BF16 && h_dtype == GI_F32 && mid_dtype == GI_F32) LAUNCH(bf16_t, float, float);
    else return gi_fail("experts_gate_up: dtypes (%d, %d, %d) are not served", w_dtype, h_dtype, mid_dtype);
#undef LAUNCH
    GI_CHECK_LAUNCH("experts_gate_up");
    return 0;
}

GI_API int gi_experts_down(const void* mid, int mid_dtype, long ldm, const void* w_down, int w_dtype, const int* ids, const float* weights, int weigh_output,
                           float* x, long ldx, int accumulate, int n_rows, int top, int width, int ff, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && top > 0 && width > 0 && ff > 0 && ldx >= width && ldm >= ff, "experts_down: bad sizes (rows %d, top %d, width %d, ff %d)", n_rows, top, width, ff);
    dim3 grid(n_rows, (width + 3) / 4);
    GI_REQUIRE(grid.y <= 65535, "experts_down: rows too wide");
#define LAUNCH(TW, TM) experts_down_kernel<TW, TM><<<grid, 256, 0, stream>>>((const TM*)mid, ldm, (const TW*)w_down, ids, weights, weigh_output, top, x, ldx, width, ff, accumulate)
    if (w_dtype == GI_BF16 && mid_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t);
    else if (w_dtype == GI_F32 && mid_dtype == GI_F32) LAUNCH(float, float);
    else if (w_dtype == GI_BF16 && mid_dtype == GI_F32) LAUNCH(bf16_t, float);
    else return gi_fail("experts_down: dtypes (%d, %d) are not served", w_dtype, mid_dtype);
#undef LAUNCH
    GI_CHECK_LAUNCH("experts_down");
    return 0;
}
