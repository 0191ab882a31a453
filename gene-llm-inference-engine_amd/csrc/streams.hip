// Several copies of the residual stream ("streams"), and the blend of a row with the row before it.
//
// A model may carry n copies x_0 .. x_(n-1) of the residual stream, laid side by side in a row: x [rows, n * width], float32.
// A half of a layer reads a weighted sum of the copies and writes its result back into every copy while the copies are mixed
// among themselves:
//
//   gi_streams_spread      every copy <- the same rows (the model's start)
//   gi_streams_norm_shift  u = sum_s read[s] x_s (read == nullptr: the plain sum);  h = norm_weight * u / sqrt(mean(u^2) + eps)
//                          (norm_weight == nullptr: h = u);  with `shift` [width]:  out = h + (h_before - h) * shift, where h_before is
//                          the h of the request's row before this one (zeros at position 0), else out = h
//   gi_streams_write       x_t <- sum_s mix[s, t] x_s + mult * write[t] * y, all copies at once from the old ones
//                          (mix == nullptr: x_t <- x_t + mult * write[t] * y)
//
// The row before a row is the step's previous row if that belongs to the same request at the position before; otherwise it was
// the last row of an earlier step, whose h the request's state slot holds (`state` [slots, width], float32).  The workgroup of a
// row makes the h of the row before it anew from that row's x (the same sums in the same order: the same bits) rather than wait
// for another workgroup.  `mode` bit 0: write `out`; bit 1: the last row of every request in the step writes its h into the
// request's slot.  A step whose requests bring one row each may do both in one launch (a row reads its slot before it writes it);
// a step with longer portions launches twice, mode 1 and then mode 2, since the first row of a portion reads the slot that the
// portion's last row writes.
//
//   gi_head_gate           a [rows, heads * vd] : head h of row t multiplied by sigmoid(gate[t, h])
//   gi_add_rows_gated      x[t] += sigmoid(g[t]) * y[t]
#include "common.h"

namespace {

constexpr int MAX_STREAMS = 16;

__global__ __launch_bounds__(256) void streams_spread_kernel(const float* __restrict__ x0, long ld0, float* __restrict__ x, long ldx, int n, int width) {
    const size_t t = blockIdx.x;
    const int d = blockIdx.y * 256 + threadIdx.x;
    if (d >= width) return;
    const float v = x0[t * ld0 + d];
    for (int s = 0; s < n; ++s) x[t * ldx + (size_t)s * width + d] = v;
}

// u[d] of one row, the copies in their order.
__device__ __forceinline__ float read_sum(const float* __restrict__ row, int n, int width, const float* w, int d) {
    float u = 0.f;
    if (w != nullptr) {
        for (int s = 0; s < n; ++s) u = fmaf(w[s], row[(size_t)s * width + d], u);
    } else {
        for (int s = 0; s < n; ++s) u += row[(size_t)s * width + d];
    }
    return u;
}

template <typename TW, typename TO>
__global__ __launch_bounds__(256) void streams_norm_shift_kernel(const float* __restrict__ x, long ldx, int n, int width, const float* __restrict__ read,
                                                                const TW* __restrict__ norm_w, float eps, const float* __restrict__ shift,
                                                                float* __restrict__ state, long state_stride, const int* __restrict__ pos,
                                                                const int* __restrict__ slot, TO* __restrict__ out, long ldo, int n_rows, int mode) {
    __shared__ float red[4];
    __shared__ float w_s[MAX_STREAMS];
    const int t = blockIdx.x;
    const bool shifts = shift != nullptr;
    bool last = false, before_in_step = false, before_in_state = false;
    if (shifts) {
        const int p = pos[t], sl = slot[t];
        last = t == n_rows - 1 || slot[t + 1] != sl || pos[t + 1] != p + 1;
        before_in_step = p > 0 && t > 0 && slot[t - 1] == sl && pos[t - 1] == p - 1;
        before_in_state = p > 0 && !before_in_step;
    }
    const bool writes_out = mode & 1, writes_state = shifts && (mode & 2) && last;
    if (!writes_out && !writes_state) return;
    if (read != nullptr && threadIdx.x < n) w_s[threadIdx.x] = read[threadIdx.x];
    __syncthreads();
    const float* w = read != nullptr ? w_s : nullptr;
    const float* row = x + (size_t)t * ldx;
    const float* row_b = row - ldx;
    const bool both = writes_out && before_in_step;
    float r = 1.f, r_b = 1.f;
    if (norm_w != nullptr) {
        float ss = 0.f, ss_b = 0.f;
        for (int d = threadIdx.x; d < width; d += 256) {
            const float u = read_sum(row, n, width, w, d);
            ss = fmaf(u, u, ss);
            if (both) {
                const float ub = read_sum(row_b, n, width, w, d);
                ss_b = fmaf(ub, ub, ss_b);
            }
        }
        r = 1.0f / sqrtf(block_sum<256>(ss, red) / (float)width + eps);
        if (both) r_b = 1.0f / sqrtf(block_sum<256>(ss_b, red) / (float)width + eps);
    }
    const int sl = shifts ? slot[t] : 0;
    for (int d = threadIdx.x; d < width; d += 256) {
        const float g = norm_w != nullptr ? load_f32(norm_w, d) : 1.f;
        float h = read_sum(row, n, width, w, d);
        if (norm_w != nullptr) h = g * (r * h);
        if (writes_out) {
            float o = h;
            if (shifts) {
                float hb = 0.f;
                if (before_in_step) {
                    hb = read_sum(row_b, n, width, w, d);
                    if (norm_w != nullptr) hb = g * (r_b * hb);
                } else if (before_in_state) {
                    hb = state[(size_t)sl * state_stride + d];
                }
                o = fmaf(hb - h, shift[d], h);
            }
            store_f32(out + (size_t)t * ldo, d, o);
        }
        if (writes_state) state[(size_t)sl * state_stride + d] = h;
    }
}

__global__ __launch_bounds__(256) void streams_write_kernel(float* __restrict__ x, long ldx, int n, int width, const float* __restrict__ y, long ldy,
                                                           const float* __restrict__ mix, const float* __restrict__ write, float mult) {
    __shared__ float m_s[MAX_STREAMS * MAX_STREAMS];
    __shared__ float o_s[MAX_STREAMS];
    if (mix != nullptr)
        for (int i = threadIdx.x; i < n * n; i += 256) m_s[i] = mix[i];
    if (threadIdx.x < n) o_s[threadIdx.x] = write != nullptr ? mult * write[threadIdx.x] : mult;
    __syncthreads();
    const size_t t = blockIdx.x;
    const int d = blockIdx.y * 256 + threadIdx.x;
    if (d >= width) return;
    float* row = x + t * ldx + d;
    const float v = y[t * ldy + d];
    float old[MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < MAX_STREAMS; ++s) old[s] = s < n ? row[(size_t)s * width] : 0.f;
#pragma unroll
    for (int to = 0; to < MAX_STREAMS; ++to) {
        if (to < n) {
            float a;
            if (mix != nullptr) {
                a = 0.f;
#pragma unroll
                for (int s = 0; s < MAX_STREAMS; ++s)
                    if (s < n) a = fmaf(m_s[s * n + to], old[s], a);
            } else {
                a = old[to];
            }
            row[(size_t)to * width] = fmaf(o_s[to], v, a);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(T* __restrict__ a, long lda, const float* __restrict__ gate, long ldg, int n_heads, int vd) {
    const size_t t = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= n_heads * vd) return;
    const float g = 1.0f / (1.0f + expf(-gate[t * ldg + c / vd]));
    store_f32(a + t * lda, c, g * load_f32(a + t * lda, c));
}

__global__ __launch_bounds__(256) void add_rows_gated_kernel(float* __restrict__ x, long ldx, const float* __restrict__ y, long ldy, const float* __restrict__ g, long ldg,
                                                            int width) {
    const size_t t = blockIdx.x;
    const int d = blockIdx.y * 256 + threadIdx.x;
    if (d >= width) return;
    const float s = 1.0f / (1.0f + expf(-g[t * ldg]));
    x[t * ldx + d] = fmaf(s, y[t * ldy + d], x[t * ldx + d]);
}

}  // namespace

GI_API int gi_streams_max() { return MAX_STREAMS; }

GI_API int gi_streams_spread(const float* x0, long ld0, float* x, long ldx, int n_rows, int n, int width, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n > 0 && width > 0 && ld0 >= width && ldx >= (long)n * width, "streams_spread: bad sizes (rows %d, %d copies of %d)", n_rows, n, width);
    dim3 grid(n_rows, (width + 255) / 256);
    GI_REQUIRE(grid.y <= 65535, "streams_spread: rows too long");
    streams_spread_kernel<<<grid, 256, 0, stream>>>(x0, ld0, x, ldx, n, width);
    GI_CHECK_LAUNCH("streams_spread");
    return 0;
}

GI_API int gi_streams_norm_shift(const float* x, long ldx, int n, int width, const float* read, const void* norm_w, int w_dtype, float eps, const float* shift,
                                 float* state, long state_stride, const int* pos, const int* slot, void* out, int out_dtype, long ldo, int n_rows, int mode,
                                 hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n > 0 && n <= MAX_STREAMS && width > 0 && ldx >= (long)n * width && ldo >= width, "streams_norm_shift: bad sizes (rows %d, %d copies of %d)",
               n_rows, n, width);
    GI_REQUIRE(mode >= 1 && mode <= 3 && ((mode & 1) == 0 || out != nullptr), "streams_norm_shift: mode %d", mode);
    GI_REQUIRE(shift != nullptr ? (state != nullptr && pos != nullptr && slot != nullptr && state_stride >= width) : mode == 1,
               "streams_norm_shift: a blend with the row before needs the state slots, positions and slots; without one there is no state to write");
#define LAUNCH(TW, TO)                                                                                                                                    \
    streams_norm_shift_kernel<TW, TO><<<n_rows, 256, 0, stream>>>(x, ldx, n, width, read, (const TW*)norm_w, eps, shift, state, state_stride, pos, slot, \
                                                                  (TO*)out, ldo, n_rows, mode)
    if (w_dtype == GI_F32 && out_dtype == GI_F32) LAUNCH(float, float);
    else if (w_dtype == GI_F32 && out_dtype == GI_BF16) LAUNCH(float, bf16_t);
    else if (w_dtype == GI_BF16 && out_dtype == GI_F32) LAUNCH(bf16_t, float);
    else if (w_dtype == GI_BF16 && out_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t);
    else return gi_fail("streams_norm_shift: unknown dtypes %d, %d", w_dtype, out_dtype);
#undef LAUNCH
    GI_CHECK_LAUNCH("streams_norm_shift");
    return 0;
}

GI_API int gi_streams_write(float* x, long ldx, int n, int width, const float* y, long ldy, const float* mix, const float* write, float mult, int n_rows,
                            hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n > 0 && n <= MAX_STREAMS && width > 0 && ldx >= (long)n * width && ldy >= width, "streams_write: bad sizes (rows %d, %d copies of %d)",
               n_rows, n, width);
    dim3 grid(n_rows, (width + 255) / 256);
    GI_REQUIRE(grid.y <= 65535, "streams_write: rows too long");
    streams_write_kernel<<<grid, 256, 0, stream>>>(x, ldx, n, width, y, ldy, mix, write, mult);
    GI_CHECK_LAUNCH("streams_write");
    return 0;
}

GI_API int gi_head_gate(void* a, int a_dtype, long lda, const float* gate, long ldg, int n_rows, int n_heads, int vd, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_heads > 0 && vd > 0 && lda >= (long)n_heads * vd && ldg >= n_heads, "head_gate: bad sizes (rows %d, %d heads of %d)", n_rows, n_heads, vd);
    dim3 grid(n_rows, (n_heads * vd + 255) / 256);
    GI_REQUIRE(grid.y <= 65535, "head_gate: rows too long");
    if (a_dtype == GI_F32) head_gate_kernel<float><<<grid, 256, 0, stream>>>((float*)a, lda, gate, ldg, n_heads, vd);
    else if (a_dtype == GI_BF16) head_gate_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)a, lda, gate, ldg, n_heads, vd);
    else return gi_fail("head_gate: unknown dtype %d", a_dtype);
    GI_CHECK_LAUNCH("head_gate");
    return 0;
}

GI_API int gi_add_rows_gated(float* x, long ldx, const float* y, long ldy, const float* g, long ldg, int n_rows, int width, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && width > 0 && ldx >= width && ldy >= width && ldg >= 1, "add_rows_gated: bad sizes (rows %d, width %d)", n_rows, width);
    dim3 grid(n_rows, (width + 255) / 256);
    GI_REQUIRE(grid.y <= 65535, "add_rows_gated: rows too long");
    add_rows_gated_kernel<<<grid, 256, 0, stream>>>(x, ldx, y, ldy, g, ldg, width);
    GI_CHECK_LAUNCH("add_rows_gated");
    return 0;
}
