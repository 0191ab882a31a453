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
//   gi_streams_write_norm  the same and, of the new copies, what the layer's next half reads: norm(sum_t read[t] x_t), in one kernel
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

// The same in one walk over the row, four neighbouring channels a thread and up to MAXC such pieces a thread kept in registers
// (widths up to 1024 MAXC, a multiple of 4): the sums u of the row (and of the row before it, where the blend needs that) are made
// once, squared and added up, and then normed, blended and stored.
constexpr int MAXC = 8;
__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
// NS > 0: the number of copies is known where the kernel is compiled (1, 2 or 4: all of a row's loads go out at once, no loop over
// them); NS = 0: any number.  The sums are the same numbers in the same order either way.
template <int NS>
__device__ __forceinline__ float4 read_sum4(const float* __restrict__ row, int n, int width, const float* w, int d) {
    float4 u = {0.f, 0.f, 0.f, 0.f};
    if constexpr (NS > 0) {
        float4 v[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s) v[s] = ld4(row + (size_t)s * width + d);
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            if (w != nullptr) { u.x = fmaf(w[s], v[s].x, u.x); u.y = fmaf(w[s], v[s].y, u.y); u.z = fmaf(w[s], v[s].z, u.z); u.w = fmaf(w[s], v[s].w, u.w); }
            else { u.x += v[s].x; u.y += v[s].y; u.z += v[s].z; u.w += v[s].w; }
        }
    } else {
        for (int s = 0; s < n; ++s) {
            const float4 v = ld4(row + (size_t)s * width + d);
            if (w != nullptr) { u.x = fmaf(w[s], v.x, u.x); u.y = fmaf(w[s], v.y, u.y); u.z = fmaf(w[s], v.z, u.z); u.w = fmaf(w[s], v.w, u.w); }
            else { u.x += v.x; u.y += v.y; u.z += v.z; u.w += v.w; }
        }
    }
    return u;
}
__device__ __forceinline__ float squares4(const float4 u, float ss) { return fmaf(u.w, u.w, fmaf(u.z, u.z, fmaf(u.y, u.y, fmaf(u.x, u.x, ss)))); }
template <typename TW>
__device__ __forceinline__ float4 weights4(const TW* w, int d) {
    if (w == nullptr) return float4{1.f, 1.f, 1.f, 1.f};
    return float4{load_f32(w, d), load_f32(w, d + 1), load_f32(w, d + 2), load_f32(w, d + 3)};
}
__device__ __forceinline__ void store4(float* p, const float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, const float4 v) { *reinterpret_cast<uint2*>(p) = uint2{f32x2_to_bf16x2(v.x, v.y), f32x2_to_bf16x2(v.z, v.w)}; }

template <typename TW, typename TO, int NS>
__global__ __launch_bounds__(256) void streams_norm_shift_fast_kernel(const float* __restrict__ x, long ldx, int n, int width, const float* __restrict__ read,
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
    float4 u[MAXC], ub[MAXC];
    float ss = 0.f, ss_b = 0.f;
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        const int d = 4 * (threadIdx.x + 256 * i);
        if (d < width) {
            u[i] = read_sum4<NS>(row, n, width, w, d);
            ss = squares4(u[i], ss);
            if (both) {
                ub[i] = read_sum4<NS>(row_b, n, width, w, d);
                ss_b = squares4(ub[i], ss_b);
            }
        }
    }
    float r = 1.f, r_b = 1.f;
    if (norm_w != nullptr) {
        r = 1.0f / sqrtf(block_sum<256>(ss, red) / (float)width + eps);
        if (both) r_b = 1.0f / sqrtf(block_sum<256>(ss_b, red) / (float)width + eps);
    }
    const int sl = shifts ? slot[t] : 0;
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        const int d = 4 * (threadIdx.x + 256 * i);
        if (d < width) {
            const float4 g = weights4(norm_w, d);
            float4 h = u[i];
            if (norm_w != nullptr) h = float4{g.x * (r * h.x), g.y * (r * h.y), g.z * (r * h.z), g.w * (r * h.w)};
            if (writes_out) {
                float4 o = h;
                if (shifts) {
                    float4 hb = {0.f, 0.f, 0.f, 0.f};
                    if (before_in_step) {
                        hb = ub[i];
                        if (norm_w != nullptr) hb = float4{g.x * (r_b * hb.x), g.y * (r_b * hb.y), g.z * (r_b * hb.z), g.w * (r_b * hb.w)};
                    } else if (before_in_state) {
                        hb = ld4(state + (size_t)sl * state_stride + d);
                    }
                    const float4 sh = ld4(shift + d);
                    o = float4{fmaf(hb.x - h.x, sh.x, h.x), fmaf(hb.y - h.y, sh.y, h.y), fmaf(hb.z - h.z, sh.z, h.z), fmaf(hb.w - h.w, sh.w, h.w)};
                }
                store4(out + (size_t)t * ldo + d, o);
            }
            if (writes_state) store4(state + (size_t)sl * state_stride + d, h);
        }
    }
}

// A half's result written into the copies and, on the way, what the layer's next half reads of them: the copies of a row become
// x_t <- sum_s mix[s, t] x_s + mult * write[t] * y, and out = norm_w * u / sqrt(mean(u^2) + eps) with u = sum_t read[t] x_t of the new
// copies.  Up to 8 copies, widths as above.
constexpr int FUSED_MAX_STREAMS = 8;
template <typename TW, typename TO, int NS>
__global__ __launch_bounds__(256) void streams_write_norm_kernel(float* __restrict__ x, long ldx, int n, int width, const float* __restrict__ y, long ldy,
                                                                const float* __restrict__ mix, const float* __restrict__ write, float mult,
                                                                const float* __restrict__ read, const TW* __restrict__ norm_w, float eps, TO* __restrict__ out, long ldo) {
    __shared__ float red[4];
    __shared__ float m_s[FUSED_MAX_STREAMS * FUSED_MAX_STREAMS];
    __shared__ float o_s[FUSED_MAX_STREAMS], r_s[FUSED_MAX_STREAMS];
    if (mix != nullptr)
        for (int i = threadIdx.x; i < n * n; i += 256) m_s[i] = mix[i];
    if (threadIdx.x < n) {
        o_s[threadIdx.x] = write != nullptr ? mult * write[threadIdx.x] : mult;
        r_s[threadIdx.x] = read != nullptr ? read[threadIdx.x] : 1.f;
    }
    __syncthreads();
    float* row = x + (size_t)blockIdx.x * ldx;
    const float* yr = y + (size_t)blockIdx.x * ldy;
    float4 u[MAXC];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        const int d = 4 * (threadIdx.x + 256 * i);
        if (d < width) {
            constexpr int MOST = NS > 0 ? NS : FUSED_MAX_STREAMS;          // (NS > 0: the number of copies, known where the kernel is compiled)
            float4 old[MOST];
#pragma unroll
            for (int s = 0; s < MOST; ++s)
                if (NS > 0 || s < n) old[s] = ld4(row + (size_t)s * width + d);
            const float4 v = ld4(yr + d);
            float4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int to = 0; to < MOST; ++to) {
                if (NS > 0 || to < n) {
                    float4 a;
                    if (mix != nullptr) {
                        a = float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int s = 0; s < MOST; ++s)
                            if (NS > 0 || s < n) {
                                const float m = m_s[s * n + to];
                                a.x = fmaf(m, old[s].x, a.x); a.y = fmaf(m, old[s].y, a.y); a.z = fmaf(m, old[s].z, a.z); a.w = fmaf(m, old[s].w, a.w);
                            }
                    } else {
                        a = old[to];
                    }
                    const float o = o_s[to], rd = r_s[to];
                    a = float4{fmaf(o, v.x, a.x), fmaf(o, v.y, a.y), fmaf(o, v.z, a.z), fmaf(o, v.w, a.w)};
                    store4(row + (size_t)to * width + d, a);
                    acc = float4{fmaf(rd, a.x, acc.x), fmaf(rd, a.y, acc.y), fmaf(rd, a.z, acc.z), fmaf(rd, a.w, acc.w)};
                }
            }
            u[i] = acc;
            ss = squares4(acc, ss);
        }
    }
    const float r = 1.0f / sqrtf(block_sum<256>(ss, red) / (float)width + eps);
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        const int d = 4 * (threadIdx.x + 256 * i);
        if (d < width) {
            const float4 g = weights4(norm_w, d);
            store4(out + (size_t)blockIdx.x * ldo + d, float4{g.x * (r * u[i].x), g.y * (r * u[i].y), g.z * (r * u[i].z), g.w * (r * u[i].w)});
        }
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
    // one walk with the row in registers where the sizes and addresses allow it, else the kernel that makes every sum twice; which
    // of the two serves is a matter of the sizes alone, so a row's numbers never depend on what else the step holds
    const bool fast = width % 4 == 0 && width <= 1024 * MAXC && ldx % 4 == 0 && ldo % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0 &&
                      (shift == nullptr || (((uintptr_t)shift & 15) == 0 && ((uintptr_t)state & 15) == 0 && state_stride % 4 == 0));
#define FAST(TW, TO, NS)                                                                                                                                  \
    streams_norm_shift_fast_kernel<TW, TO, NS><<<n_rows, 256, 0, stream>>>(x, ldx, n, width, read, (const TW*)norm_w, eps, shift, state, state_stride, pos, slot, \
                                                                           (TO*)out, ldo, n_rows, mode)
#define LAUNCH(TW, TO)                                                                                                                                    \
    do {                                                                                                                                                  \
        if (fast && n == 1) FAST(TW, TO, 1);                                                                                                              \
        else if (fast && n == 2) FAST(TW, TO, 2);                                                                                                         \
        else if (fast && n == 4) FAST(TW, TO, 4);                                                                                                         \
        else if (fast) FAST(TW, TO, 0);                                                                                                                   \
        else                                                                                                                                              \
            streams_norm_shift_kernel<TW, TO><<<n_rows, 256, 0, stream>>>(x, ldx, n, width, read, (const TW*)norm_w, eps, shift, state, state_stride, pos, slot, \
                                                                          (TO*)out, ldo, n_rows, mode);                                                \
    } while (0)
    if (w_dtype == GI_F32 && out_dtype == GI_F32) LAUNCH(float, float);
    else if (w_dtype == GI_F32 && out_dtype == GI_BF16) LAUNCH(float, bf16_t);
    else if (w_dtype == GI_BF16 && out_dtype == GI_F32) LAUNCH(bf16_t, float);
    else if (w_dtype == GI_BF16 && out_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t);
    else return gi_fail("streams_norm_shift: unknown dtypes %d, %d", w_dtype, out_dtype);
#undef LAUNCH
#undef FAST
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

GI_API int gi_streams_write_norm_takes(int n, int width) { return n >= 1 && n <= FUSED_MAX_STREAMS && width % 4 == 0 && width <= 1024 * MAXC ? 1 : 0; }

GI_API int gi_streams_write_norm(float* x, long ldx, int n, int width, const float* y, long ldy, const float* mix, const float* write, float mult, const float* read,
                                 const void* norm_w, int w_dtype, float eps, void* out, int out_dtype, long ldo, int n_rows, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && gi_streams_write_norm_takes(n, width) && ldx >= (long)n * width && ldy >= width && ldo >= width && norm_w != nullptr && out != nullptr,
               "streams_write_norm: bad sizes (rows %d, %d copies of %d)", n_rows, n, width);
    GI_REQUIRE(ldx % 4 == 0 && ldy % 4 == 0 && ldo % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)y & 15) == 0 && ((uintptr_t)out & 15) == 0,
               "streams_write_norm: rows must start at multiples of 16 bytes");
#define GO(TW, TO, NS) streams_write_norm_kernel<TW, TO, NS><<<n_rows, 256, 0, stream>>>(x, ldx, n, width, y, ldy, mix, write, mult, read, (const TW*)norm_w, eps, (TO*)out, ldo)
#define LAUNCH(TW, TO)                  \
    do {                                \
        if (n == 1) GO(TW, TO, 1);      \
        else if (n == 2) GO(TW, TO, 2); \
        else if (n == 4) GO(TW, TO, 4); \
        else GO(TW, TO, 0);             \
    } while (0)
    if (w_dtype == GI_F32 && out_dtype == GI_F32) LAUNCH(float, float);
    else if (w_dtype == GI_F32 && out_dtype == GI_BF16) LAUNCH(float, bf16_t);
    else if (w_dtype == GI_BF16 && out_dtype == GI_F32) LAUNCH(bf16_t, float);
    else if (w_dtype == GI_BF16 && out_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t);
    else return gi_fail("streams_write_norm: unknown dtypes %d, %d", w_dtype, out_dtype);
#undef LAUNCH
#undef GO
    GI_CHECK_LAUNCH("streams_write_norm");
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
