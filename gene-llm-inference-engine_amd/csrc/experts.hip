// A feed-forward made of many small gated feed-forwards ("experts"), of which every row uses a few, chosen by a router.
//
//   gi_route_top         the router's choice per row: scores (sigmoid of the logits, or a softmax over them), the `top` largest
//                        (the lower index wins a tie), optionally divided by their sum
//   gi_experts_gate_up   mid[(row, choice)] = act(W_gate[e] a) * (W_up[e] a), e the row's choice and a the row, multiplied by the
//                        choice's score first where the score weighs the expert's input
//   gi_experts_down      x[row] (+)= sum over the row's choices of (score, where it weighs the output) * W_down[e] mid[(row, choice)]
//
// These two walk the weights of each (row, choice) with one wave per output: the form for the few rows of decoding steps, where
// every row reads its own experts and the weights' bytes are the cost, and the form of 32-bit models.  Every sum is a lane's own
// share in a fixed order, then the lanes by a butterfly, then the choices one after the other: nothing depends on the batch.
//
//   gi_route_rows        the router's product and its choice in one: logits = W_router a per row, 32-bit sums in a fixed order; rows of
//                        the matrix behind the experts' (a gate on a shared expert, say) are multiplied along and their products kept
//
// For many (row, choice) items in bfloat16 the items are put in the order of their experts, every expert's run filled up to whole
// tiles of 128 rows, so that one launch of the matrix-core product for grouped rows (gemm_bf16.hip) serves all experts:
//   gi_experts_count     how many items chose each expert
//   gi_experts_place     every item's place in that order (an expert's items keep their order), and every tile's expert
//   gi_experts_gather    the rows of the items (times their score, where it weighs the input) at their places, as bfloat16
//   gi_experts_combine   x[row] (+)= the sum over the row's choices of the results at their places (times the score, where it
//                        weighs the output), the choices one after the other
// Nothing of this asks the host how the router chose: the launches' shapes depend on the number of items and experts alone.
#include "common.h"

namespace {

constexpr int ROUTE_PER_LANE = 16;      // experts a lane looks at: up to 1024 experts

// What the router makes of a row's logits (z: this lane's experts lane, lane + 64, ...; -inf beyond the last): the scores
// (score_kind 0: sigmoid, 1: softmax over all experts), the `top` largest (the lower index wins a tie), optionally divided by
// their sum + floor.  With n_groups > 1 the experts form that many equal groups of neighbours, a group scores what its best
// expert scores, and only experts of the `keep` best groups can be chosen (the lower group wins a tie).
__device__ __forceinline__ void choose_experts(float (&z)[ROUTE_PER_LANE], int lane, size_t t, int n_experts, int top, int score_kind, int renormalize, float floor,
                                               int n_groups, int keep, int* __restrict__ ids, float* __restrict__ weights) {
    float biggest = -INFINITY;
#pragma unroll
    for (int i = 0; i < ROUTE_PER_LANE; ++i) biggest = fmaxf(biggest, z[i]);
    float denominator = 1.0f;
    if (score_kind == 1) {
        biggest = wave_max(biggest);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < ROUTE_PER_LANE; ++i) s += lane + 64 * i < n_experts ? expf(z[i] - biggest) : 0.f;
        denominator = wave_sum(s);
    }
    if (n_groups > 1 && keep < n_groups) {
        const int per = n_experts / n_groups;
        unsigned kept = 0, taken = 0;                   // bit i: expert lane + 64 i lies in a group that is kept / has been looked at
        for (int k = 0; k < keep; ++k) {
            float best = -INFINITY;
            int at = 0x7fffffff;
#pragma unroll
            for (int i = 0; i < ROUTE_PER_LANE; ++i) {
                if (!((taken >> i) & 1u) && z[i] > best) best = z[i], at = lane + 64 * i;
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const float ob = __shfl_xor(best, off, 64);
                const int oa = __shfl_xor(at, off, 64);
                if (ob > best || (ob == best && oa < at)) best = ob, at = oa;
            }
            const int g = at / per;
#pragma unroll
            for (int i = 0; i < ROUTE_PER_LANE; ++i) {
                if ((lane + 64 * i) / per == g) kept |= 1u << i, taken |= 1u << i;
            }
        }
#pragma unroll
        for (int i = 0; i < ROUTE_PER_LANE; ++i) {
            if (!((kept >> i) & 1u)) z[i] = -INFINITY;
        }
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
        weights[t * top + lane] = renormalize ? mine / (total + floor) : mine;
    }
}

// One wave per row.
__global__ __launch_bounds__(64) void route_top_kernel(const float* __restrict__ logits, long ld, int n_experts, int top, int score_kind, int renormalize,
                                                      float floor, int n_groups, int keep, int* __restrict__ ids, float* __restrict__ weights) {
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x;
    float z[ROUTE_PER_LANE];
#pragma unroll
    for (int i = 0; i < ROUTE_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        z[i] = e < n_experts ? logits[t * ld + e] : -INFINITY;
    }
    choose_experts(z, lane, t, n_experts, top, score_kind, renormalize, floor, n_groups, keep, ids, weights);
}

// One wave per (row, choice, output j): both dot products over the row, the lanes' shares of k interleaved.
template <typename TW, typename TA, typename TO>
__global__ __launch_bounds__(256) void experts_gate_up_kernel(const TA* __restrict__ h, long ldh, const TW* __restrict__ w_gate, const TW* __restrict__ w_up,
                                                             const int* __restrict__ ids, const float* __restrict__ weights, int weigh_input,
                                                             int top, TO* __restrict__ mid, long ldm, int width, int ff, int act, float limit, int group) {
    const size_t item = blockIdx.x;                     // (row * top + choice)
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int j = blockIdx.y * 4 + wave;
    if (j >= ff) return;
    const size_t row = item / top, e = ids[item];
    const float s = weigh_input ? weights[item] : 1.0f;
    const TA* a = h + row * ldh;
    // group > 0: one stack [experts][2 ff][width] of `group` gate rows, the `group` up rows of the same outputs, and so on
    const TW* g = group > 0 ? w_gate + (e * 2 * ff + (size_t)(j / group) * 2 * group + j % group) * (size_t)width : w_gate + (e * ff + j) * (size_t)width;
    const TW* u = group > 0 ? g + (size_t)group * width : w_up + (e * ff + j) * (size_t)width;
    float sg = 0.f, su = 0.f;
    for (int d = lane; d < width; d += 64) {
        float v = s * load_f32(a, d);
        if (sizeof(TA) == 2) v = bf16_to_f32(f32_to_bf16(v));      // rows that go into a product are stored as the product reads them
        sg = fmaf(load_f32(g, d), v, sg);
        su = fmaf(load_f32(u, d), v, su);
    }
    sg = wave_sum(sg);
    su = wave_sum(su);
    if (lane == 0) store_f32(mid + item * ldm, j, gated_act(sg, su, act, limit));
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

// The router's product and choice for one row: a workgroup of four waves; wave w makes the logits of experts w, w + 4, ..., every
// one a lane's share of the columns in their order and then the lanes by a butterfly; the first wave then chooses as
// `route_top_kernel` does.
constexpr int ROUTE_MAX_EXPERTS = 64 * ROUTE_PER_LANE;
template <typename TA, typename TW>
__global__ __launch_bounds__(256) void route_rows_kernel(const TA* __restrict__ h, long ldh, const TW* __restrict__ router, long ldr, int width, int n_experts, int top,
                                                        int score_kind, int renormalize, float floor, int n_groups, int keep, int* __restrict__ ids, float* __restrict__ weights,
                                                        float* __restrict__ logits_out, long ldl, int n_extra, float* __restrict__ extra_out, long lde) {
    __shared__ float zs[ROUTE_MAX_EXPERTS];
    const size_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const TA* a = h + t * ldh;
    for (int e = wave; e < n_experts + n_extra; e += 4) {          // (rows behind the experts': products of the same rows that are no expert's, kept for the caller)
        const TW* w = router + (size_t)e * ldr;
        // a lane takes eight neighbouring columns at a time, four such pieces asked for at once; the columns left over one by one
        float s = 0.f;
        const int whole = width & ~7;
#pragma unroll 4
        for (int d = lane * 8; d < whole; d += 512) {
            float wv[8], av[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) wv[i] = load_f32(w, d + i), av[i] = load_f32(a, d + i);
#pragma unroll
            for (int i = 0; i < 8; ++i) s = fmaf(wv[i], av[i], s);
        }
        for (int d = whole + lane; d < width; d += 64) s = fmaf(load_f32(w, d), load_f32(a, d), s);
        s = wave_sum(s);
        if (lane == 0) {
            if (e >= n_experts) extra_out[t * lde + (e - n_experts)] = s;
            else {
                zs[e] = s;
                if (logits_out != nullptr) logits_out[t * ldl + e] = s;
            }
        }
    }
    __syncthreads();
    if (wave != 0) return;
    float z[ROUTE_PER_LANE];
#pragma unroll
    for (int i = 0; i < ROUTE_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        z[i] = e < n_experts ? zs[e] : -INFINITY;
    }
    choose_experts(z, lane, t, n_experts, top, score_kind, renormalize, floor, n_groups, keep, ids, weights);
}

constexpr int EXPERT_TILE = 128;          // rows of a tile of the grouped product

__device__ __forceinline__ int wave_sum_int(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// One wave per expert: how many of the items chose it.
__global__ __launch_bounds__(256) void experts_count_kernel(const int* __restrict__ ids, int n_items, int n_experts, int* __restrict__ count) {
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (e >= n_experts) return;
    int c = 0;
    for (int i = lane; i < n_items; i += 64) c += ids[i] == e ? 1 : 0;
    c = wave_sum_int(c);
    if (lane == 0) count[e] = c;
}

// One wave per expert: where its run begins (behind the runs of the experts before it, each filled up to whole tiles), its tiles'
// entries, and its items' places in their order.  The last expert's wave also marks the tiles behind all runs as not in use.
__global__ __launch_bounds__(256) void experts_place_kernel(const int* __restrict__ ids, int n_items, int n_experts, const int* __restrict__ count,
                                                           int* __restrict__ place, int* __restrict__ tile_expert, int n_tiles) {
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (e >= n_experts) return;
    int before = 0;
    for (int o = lane; o < e; o += 64) before += (count[o] + EXPERT_TILE - 1) / EXPERT_TILE;
    before = wave_sum_int(before);
    const int mine = (count[e] + EXPERT_TILE - 1) / EXPERT_TILE;
    for (int j = lane; j < mine; j += 64) tile_expert[before + j] = e;
    if (e == n_experts - 1)
        for (int j = before + mine + lane; j < n_tiles; j += 64) tile_expert[j] = -1;
    int at = before * EXPERT_TILE;
    for (int i0 = 0; i0 < n_items; i0 += 64) {
        const int i = i0 + lane;
        const bool hit = i < n_items && ids[i] == e;
        const unsigned long long all = __ballot(hit);
        if (hit) place[i] = at + __popcll(all & ((1ull << lane) - 1ull));
        at += __popcll(all);
    }
}

// The row of every item at its place, times the item's score where that weighs the input, eight columns a thread.
__global__ __launch_bounds__(256) void experts_gather_kernel(const bf16_t* __restrict__ h, long ldh, const int* __restrict__ place, const float* __restrict__ weights,
                                                            int weigh_input, int top, bf16_t* __restrict__ out, long ldo, int width) {
    const size_t item = blockIdx.x;
    const bf16_t* a = h + (item / top) * ldh;
    bf16_t* o = out + (size_t)place[item] * ldo;
    const float s = weigh_input ? weights[item] : 1.0f;
    for (int c = threadIdx.x * 8; c < width; c += 256 * 8) {
        uint4 v = *reinterpret_cast<const uint4*>(a + c);
        if (weigh_input) {
            uint32_t* p = reinterpret_cast<uint32_t*>(&v);
#pragma unroll
            for (int i = 0; i < 4; ++i) p[i] = f32x2_to_bf16x2(s * __uint_as_float(p[i] << 16), s * __uint_as_float(p[i] & 0xffff0000u));
        }
        *reinterpret_cast<uint4*>(o + c) = v;
    }
}

__global__ __launch_bounds__(256) void experts_combine_kernel(const float* __restrict__ y, long ldy, const int* __restrict__ place, const float* __restrict__ weights,
                                                             int weigh_output, int top, float* __restrict__ x, long ldx, int width, int accumulate) {
    const size_t row = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= width) return;
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
        const size_t item = row * top + k;
        const float v = y[(size_t)place[item] * ldy + c];
        total += weigh_output ? weights[item] * v : v;
    }
    x[row * ldx + c] = accumulate ? x[row * ldx + c] + total : total;
}

}  // namespace

static int groups_fit(int n_experts, int top, int n_groups, int keep) {
    return n_groups >= 1 && n_experts % n_groups == 0 && keep >= 1 && keep <= n_groups && top <= keep * (n_experts / n_groups);
}

GI_API int gi_route_top(const float* logits, long ld, int n_rows, int n_experts, int top, int score_kind, int renormalize, float floor, int n_groups, int keep,
                        int* ids, float* weights, hipStream_t stream) {
    GI_REQUIRE(groups_fit(n_experts, top, n_groups, keep), "route_top: %d experts in %d groups of which %d are kept cannot give %d a row", n_experts, n_groups, keep, top);
    GI_REQUIRE(n_rows > 0 && n_experts > 0 && n_experts <= 64 * ROUTE_PER_LANE && top > 0 && top <= n_experts && top <= 64 && ld >= n_experts && (score_kind == 0 || score_kind == 1),
               "route_top: bad sizes (rows %d, experts %d, top %d)", n_rows, n_experts, top);
    route_top_kernel<<<n_rows, 64, 0, stream>>>(logits, ld, n_experts, top, score_kind, renormalize, floor, n_groups, keep, ids, weights);
    GI_CHECK_LAUNCH("route_top");
    return 0;
}

GI_API int gi_experts_gate_up(const void* h, int h_dtype, long ldh, const void* w_gate, const void* w_up, int w_dtype, const int* ids, const float* weights,
                              int weigh_input, void* mid, int mid_dtype, long ldm, int n_rows, int top, int width, int ff, int act, float limit, int group, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && top > 0 && top <= 65535 && width > 0 && ff > 0 && ldh >= width && ldm >= ff && act >= 0 && act < GI_N_ACTIVATIONS && (long)n_rows * top < (1l << 31)
               && (group == 0 ? w_up != nullptr : group > 0 && ff % group == 0),
               "experts_gate_up: bad sizes (rows %d, top %d, width %d, ff %d)", n_rows, top, width, ff);
    dim3 grid(n_rows * top, (ff + 3) / 4);
    GI_REQUIRE(grid.y <= 65535, "experts_gate_up: experts too wide");
#define LAUNCH(TW, TA, TO)                                                                                                                      \
    experts_gate_up_kernel<TW, TA, TO><<<grid, 256, 0, stream>>>((const TA*)h, ldh, (const TW*)w_gate, (const TW*)w_up, ids, weights, weigh_input, \
                                                                 top, (TO*)mid, ldm, width, ff, act, limit, group)
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

GI_API int gi_route_rows(const void* h, int h_dtype, long ldh, const void* router, int r_dtype, long ldr, int n_rows, int width, int n_experts, int top, int score_kind,
                         int renormalize, float floor, int n_groups, int keep, int* ids, float* weights, float* logits, long ldl, int n_extra, float* extra, long lde,
                         hipStream_t stream) {
    GI_REQUIRE(n_extra >= 0 && (n_extra == 0 || (extra != nullptr && lde >= n_extra)), "route_rows: %d rows behind the experts' need room for their products", n_extra);
    GI_REQUIRE(groups_fit(n_experts, top, n_groups, keep), "route_rows: %d experts in %d groups of which %d are kept cannot give %d a row", n_experts, n_groups, keep, top);
    GI_REQUIRE(n_rows > 0 && width > 0 && n_experts > 0 && n_experts <= ROUTE_MAX_EXPERTS && top > 0 && top <= n_experts && top <= 64 && ldh >= width && ldr >= width
               && (score_kind == 0 || score_kind == 1) && (logits == nullptr || ldl >= n_experts),
               "route_rows: bad sizes (rows %d, width %d, experts %d, top %d)", n_rows, width, n_experts, top);
#define LAUNCH(TA, TW) route_rows_kernel<TA, TW><<<n_rows, 256, 0, stream>>>((const TA*)h, ldh, (const TW*)router, ldr, width, n_experts, top, score_kind, renormalize, floor, n_groups, keep, ids, weights, logits, ldl, n_extra, extra, lde)
    if (h_dtype == GI_BF16 && r_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t);
    else if (h_dtype == GI_F32 && r_dtype == GI_F32) LAUNCH(float, float);
    else if (h_dtype == GI_F32 && r_dtype == GI_BF16) LAUNCH(float, bf16_t);
    else if (h_dtype == GI_BF16 && r_dtype == GI_F32) LAUNCH(bf16_t, float);
    else return gi_fail("route_rows: unknown dtypes %d, %d", h_dtype, r_dtype);
#undef LAUNCH
    GI_CHECK_LAUNCH("route_rows");
    return 0;
}

GI_API int gi_experts_tile_rows() { return EXPERT_TILE; }

// count [experts], place [items], tile_expert [n_tiles] with n_tiles >= (items + experts * (tile rows - 1)) / tile rows.
GI_API int gi_experts_place(const int* ids, int n_items, int n_experts, int* count, int* place, int* tile_expert, int n_tiles, hipStream_t stream) {
    GI_REQUIRE(n_items > 0 && n_experts > 0 && (long)n_tiles * EXPERT_TILE >= (long)n_items + (long)n_experts * (EXPERT_TILE - 1) - (EXPERT_TILE - 1),
               "experts_place: bad sizes (items %d, experts %d, tiles %d)", n_items, n_experts, n_tiles);
    experts_count_kernel<<<(n_experts + 3) / 4, 256, 0, stream>>>(ids, n_items, n_experts, count);
    GI_CHECK_LAUNCH("experts_count");
    experts_place_kernel<<<(n_experts + 3) / 4, 256, 0, stream>>>(ids, n_items, n_experts, count, place, tile_expert, n_tiles);
    GI_CHECK_LAUNCH("experts_place");
    return 0;
}

GI_API int gi_experts_gather(const void* h, long ldh, const int* place, const float* weights, int weigh_input, int n_rows, int top, void* out, long ldo, int width,
                             hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && top > 0 && width > 0 && width % 8 == 0 && ldh % 8 == 0 && ldo % 8 == 0 && ldh >= width && ldo >= width && (long)n_rows * top < (1l << 31)
               && ((uintptr_t)h & 15) == 0 && ((uintptr_t)out & 15) == 0, "experts_gather: bad sizes (rows %d, top %d, width %d)", n_rows, top, width);
    experts_gather_kernel<<<n_rows * top, 256, 0, stream>>>((const bf16_t*)h, ldh, place, weights, weigh_input, top, (bf16_t*)out, ldo, width);
    GI_CHECK_LAUNCH("experts_gather");
    return 0;
}

GI_API int gi_experts_combine(const float* y, long ldy, const int* place, const float* weights, int weigh_output, int n_rows, int top, float* x, long ldx, int width,
                              int accumulate, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && top > 0 && width > 0 && ldy >= width && ldx >= width, "experts_combine: bad sizes (rows %d, top %d, width %d)", n_rows, top, width);
    dim3 grid(n_rows, (width + 255) / 256);
    GI_REQUIRE(grid.y <= 65535, "experts_combine: rows too wide");
    experts_combine_kernel<<<grid, 256, 0, stream>>>(y, ldy, place, weights, weigh_output, top, x, ldx, width, accumulate);
    GI_CHECK_LAUNCH("experts_combine");
    return 0;
}

