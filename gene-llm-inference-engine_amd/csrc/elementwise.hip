// Row-wise kernels around the matrix products: token embedding, RMS norm, rotary angles,
// rotation + cache write, SiLU gating, row gather.  All arithmetic is 32-bit (angles 64-bit);
// only what is loaded or stored may be bfloat16.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";

int gi_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return -1;
}

GI_API const char* gi_last_error() { return g_error; }

// Compute units of the current device, asked for once per device; where no device answers, those of an MI355X.  Dispatch
// rules that speak of "one round of workgroups" or "three quarters of the chip" are stated in terms of this number.
GI_API int gi_compute_units() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();
        return 256;
    }
    int n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
    if (n > 0) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        n = 256;
    }
    __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
    return n;
}

GI_API int gi_device_arch(char* out, int cap) {
    hipDeviceProp_t p;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&p, dev) != hipSuccess) return gi_fail("no HIP device");
    snprintf(out, cap, "%s", p.gcnArchName);
    return 0;
}

// ------------------------------------------------------------------------------------- embedding
// x[t, :] = table[tokens[t], :], widened to 32-bit.  Reference: src/gpu/device_kernels.inc:37-51.
template <typename TT>
__global__ void embed_kernel(const TT* __restrict__ table, const int* __restrict__ tokens, float* __restrict__ x, int dim) {
    const int t = blockIdx.x;
    const TT* row = table + (size_t)tokens[t] * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) x[(size_t)t * dim + d] = load_f32(row, d);
}

GI_API int gi_embed(const void* table, int table_dtype, const int* tokens, float* x, int n_rows, int dim, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0, "embed: n_rows %d and dim %d must be positive", n_rows, dim);
    if (table_dtype == GI_F32)
        embed_kernel<float><<<n_rows, 256, 0, stream>>>((const float*)table, tokens, x, dim);
    else if (table_dtype == GI_BF16)
        embed_kernel<bf16_t><<<n_rows, 256, 0, stream>>>((const bf16_t*)table, tokens, x, dim);
    else
        return gi_fail("embed: unknown table dtype %d", table_dtype);
    GI_CHECK_LAUNCH("embed");
    return 0;
}

// The same for a step of a few rows whose first norm the product behind it finishes (see the products' `NormIn`): beside x the
// row goes out times the norm's weights in bfloat16, and its sum of squares as one number.
template <typename TT>
__global__ __launch_bounds__(256) void embed_handing_kernel(const TT* __restrict__ table, const int* __restrict__ tokens, float* __restrict__ x, int dim,
                                                            const float* __restrict__ g, bf16_t* __restrict__ scaled, float* __restrict__ squares) {
    __shared__ float red[4];
    const int t = blockIdx.x;
    const TT* row = table + (size_t)tokens[t] * dim;
    float sum = 0.f;
    if (dim % 4 == 0 && (((uintptr_t)table | (uintptr_t)x | (uintptr_t)g | (uintptr_t)scaled) & 15) == 0) {      // four neighbouring channels a thread
        for (int d = threadIdx.x * 4; d < dim; d += 1024) {
            float v[4];
            if constexpr (sizeof(TT) == 2) {
                const uint2 raw = *reinterpret_cast<const uint2*>(row + d);
                v[0] = __uint_as_float(raw.x << 16); v[1] = __uint_as_float(raw.x & 0xffff0000u);
                v[2] = __uint_as_float(raw.y << 16); v[3] = __uint_as_float(raw.y & 0xffff0000u);
            } else {
                const float4 raw = *reinterpret_cast<const float4*>(row + d);
                v[0] = raw.x; v[1] = raw.y; v[2] = raw.z; v[3] = raw.w;
            }
            const float4 gd = *reinterpret_cast<const float4*>(g + d);
            *reinterpret_cast<float4*>(x + (size_t)t * dim + d) = float4{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<uint2*>(scaled + (size_t)t * dim + d) = uint2{f32x2_to_bf16x2(gd.x * v[0], gd.y * v[1]), f32x2_to_bf16x2(gd.z * v[2], gd.w * v[3])};
            sum += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
        }
    } else {
        for (int d = threadIdx.x; d < dim; d += 256) {
            const float v = load_f32(row, d);
            x[(size_t)t * dim + d] = v;
            scaled[(size_t)t * dim + d] = f32_to_bf16(g[d] * v);
            sum = fmaf(v, v, sum);
        }
    }
    sum = block_sum<256>(sum, red);
    if (threadIdx.x == 0) squares[t] = sum;
}

GI_API int gi_embed_handing(const void* table, int table_dtype, const int* tokens, float* x, int n_rows, int dim, const float* g, void* scaled,
                            float* squares, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0 && g != nullptr && scaled != nullptr && squares != nullptr, "embed: n_rows %d and dim %d must be positive, and the norm's operands given", n_rows, dim);
    if (table_dtype == GI_F32)
        embed_handing_kernel<float><<<n_rows, 256, 0, stream>>>((const float*)table, tokens, x, dim, g, (bf16_t*)scaled, squares);
    else if (table_dtype == GI_BF16)
        embed_handing_kernel<bf16_t><<<n_rows, 256, 0, stream>>>((const bf16_t*)table, tokens, x, dim, g, (bf16_t*)scaled, squares);
    else
        return gi_fail("embed: unknown table dtype %d", table_dtype);
    GI_CHECK_LAUNCH("embed");
    return 0;
}

// -------------------------------------------------------------------------------------- RMS norm
// out = w * (x * rsqrt(mean(x^2) + eps)), one workgroup per row; the sum of squares is taken in
// 32-bit in an order that depends on the row's length only.  Reference: src/kernels/kernels.cpp:72-83.
template <typename TW, typename TO>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const TW* __restrict__ w, TO* __restrict__ out, int dim, float eps,
                               size_t x_stride, size_t out_stride) {
    __shared__ float red[4];
    const float* xr = x + (size_t)blockIdx.x * x_stride;
    TO* orow = out + (size_t)blockIdx.x * out_stride;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) ss = fmaf(xr[d], xr[d], ss);
    ss = block_sum<256>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)dim + eps);
    for (int d = threadIdx.x; d < dim; d += 256) store_f32(orow, d, load_f32(w, d) * (scale * xr[d]));
}

// The same for rows whose length is a multiple of 4 and at most 4096, 16-byte aligned: every thread
// loads its (at most four) groups of four values at once and keeps them for the second pass, so the
// kernel waits for memory once.  `rows` (optional) gathers the input rows.
__device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) { *reinterpret_cast<float4*>(p) = float4{a, b, c, d}; }
__device__ __forceinline__ void store4(bf16_t* p, float a, float b, float c, float d) {
    *reinterpret_cast<uint2*>(p) = uint2{(uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16), (uint32_t)f32_to_bf16(c) | ((uint32_t)f32_to_bf16(d) << 16)};
}
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    return float4{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u)};
}

template <typename TW, typename TO>
__global__ __launch_bounds__(256) void rmsnorm_fast_kernel(const float* __restrict__ x, const int* __restrict__ rows, const TW* __restrict__ w,
                                                          TO* __restrict__ out, int dim, float eps, size_t x_stride, size_t out_stride) {
    __shared__ float red[4];
    const float* xr = x + (size_t)(rows ? rows[blockIdx.x] : blockIdx.x) * x_stride;
    TO* orow = out + (size_t)blockIdx.x * out_stride;
    const int n4 = dim / 4;
    float4 v[4], wv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = threadIdx.x + 256 * i;
        v[i] = c < n4 ? load4(xr + 4 * c) : float4{0.f, 0.f, 0.f, 0.f};
        wv[i] = c < n4 ? load4(w + 4 * c) : float4{0.f, 0.f, 0.f, 0.f};
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        ss = fmaf(v[i].x, v[i].x, ss); ss = fmaf(v[i].y, v[i].y, ss); ss = fmaf(v[i].z, v[i].z, ss); ss = fmaf(v[i].w, v[i].w, ss);
    }
    ss = block_sum<256>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)dim + eps);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = threadIdx.x + 256 * i;
        if (c < n4) store4(orow + 4 * c, wv[i].x * (scale * v[i].x), wv[i].y * (scale * v[i].y), wv[i].z * (scale * v[i].z), wv[i].w * (scale * v[i].w));
    }
}

// rows != nullptr: out[i] = norm(x[rows[i]]) (needs the fast kernel's conditions: dim a multiple of 4, at most 4096, aligned rows).
GI_API int gi_rmsnorm(const float* x, const int* rows, const void* w, int w_dtype, void* out, int out_dtype, int n_rows, int dim, float eps,
                      long x_stride, long out_stride, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0, "rmsnorm: n_rows %d and dim %d must be positive", n_rows, dim);
    GI_REQUIRE(x_stride >= dim && out_stride >= dim, "rmsnorm: row strides must be at least dim");
    const bool fast = dim % 4 == 0 && dim <= 4096 && x_stride % 4 == 0 && out_stride % 4 == 0 && ((uintptr_t)x & 15) == 0 &&
                      ((uintptr_t)w & 15) == 0 && ((uintptr_t)out & 15) == 0;
    GI_REQUIRE(rows == nullptr || fast, "rmsnorm: gathering rows needs a row length that is a multiple of 4 and at most 4096, and aligned operands");
#define LAUNCH(TW, TO)                                                                                                                   \
    do {                                                                                                                                 \
        if (fast) rmsnorm_fast_kernel<TW, TO><<<n_rows, 256, 0, stream>>>(x, rows, (const TW*)w, (TO*)out, dim, eps, (size_t)x_stride, (size_t)out_stride); \
        else rmsnorm_kernel<TW, TO><<<n_rows, 256, 0, stream>>>(x, (const TW*)w, (TO*)out, dim, eps, (size_t)x_stride, (size_t)out_stride);              \
    } while (0)
    if (w_dtype == GI_F32 && out_dtype == GI_F32) LAUNCH(float, float);
    else if (w_dtype == GI_F32 && out_dtype == GI_BF16) LAUNCH(float, bf16_t);
    else if (w_dtype == GI_BF16 && out_dtype == GI_F32) LAUNCH(bf16_t, float);
    else if (w_dtype == GI_BF16 && out_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t);
    else return gi_fail("rmsnorm: unknown dtypes %d, %d", w_dtype, out_dtype);
#undef LAUNCH
    GI_CHECK_LAUNCH("rmsnorm");
    return 0;
}

// -------------------------------------------------------------------------------- rotary angles
// cos and sin of pos * f_k for every row, the angle taken in 64-bit: a 32-bit angle loses digits
// at large positions (reference: src/kernels/kernels.cpp:145-161).  `magnitude` multiplies both (1 for a plain rotation; rules
// that stretch the frequencies for longer contexts lengthen the turned vectors a little as well).
__global__ void rope_cos_sin_kernel(const int* __restrict__ pos, const double* __restrict__ inv_freq, float* __restrict__ cos_out,
                                    float* __restrict__ sin_out, int n_rows, int half, float magnitude) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_rows * half) return;
    const double a = (double)pos[i / half] * inv_freq[i % half];
    cos_out[i] = (float)cos(a) * magnitude;
    sin_out[i] = (float)sin(a) * magnitude;
}

GI_API int gi_rope_cos_sin(const int* pos, const double* inv_freq, float* cos_out, float* sin_out, int n_rows, int half, float magnitude,
                           hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && half > 0, "rope_cos_sin: n_rows %d and half %d must be positive", n_rows, half);
    const int n = n_rows * half;
    rope_cos_sin_kernel<<<(n + 255) / 256, 256, 0, stream>>>(pos, inv_freq, cos_out, sin_out, n_rows, half, magnitude);
    GI_CHECK_LAUNCH("rope_cos_sin");
    return 0;
}

// ---------------------------------------------------------------- rotation and cache write, fused
// For row t at position pos[t] of the request in slot[t]:
//   q heads are rotated and written to q_out [n_rows, n_heads*hd];
//   k heads are rotated and, with the v heads as they are, written into the page
//   table[slot[t]][pos / page_size] at place pos % page_size.
// Pairs are (k, k + hd/2): a' = a*cos - b*sin, b' = a*sin + b*cos (src/kernels/kernels.cpp:165-180).
// Cache of one layer: per page the keys [kv_head][place][hd], then the values transposed
// [kv_head][hd][place] (so that consecutive positions of one value channel are contiguous, which is
// what the matrix instructions of the attention kernels load).  cos == nullptr means no rotation.
// k == nullptr means the layer reads another layer's cache and writes none.
template <typename TQ, typename TC>
__global__ void rope_store_kernel(const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v, long ldq, long ldk,
                                  long ldv, const float* __restrict__ cos_t, const float* __restrict__ sin_t, const int* __restrict__ pos,
                                  const int* __restrict__ slot, const int* __restrict__ table, int table_stride, TQ* __restrict__ q_out,
                                  TC* __restrict__ cache, long page_stride, int page_size, int n_heads, int n_kv, int hd) {
    // One thread per pair: items 0 .. n_heads*half-1 are query pairs, the rest key pairs (which also carry the two values).
    const int t = blockIdx.x, half = hd / 2;
    const int i = blockIdx.y * blockDim.x + threadIdx.x;
    const int n_q_items = n_heads * half, n_k_items = k ? n_kv * half : 0;
    if (i >= n_q_items + n_k_items) return;
    const bool is_q = i < n_q_items;
    const int j = is_q ? i : i - n_q_items, h = j / half, kk = j % half;
    const float cc = cos_t ? cos_t[(size_t)t * half + kk] : 1.f, ss = sin_t ? sin_t[(size_t)t * half + kk] : 0.f;
    if (is_q) {
        const float a = q[(size_t)t * ldq + h * hd + kk], b = q[(size_t)t * ldq + h * hd + kk + half];
        store_f32(q_out, (size_t)t * n_heads * hd + h * hd + kk, a * cc - b * ss);
        store_f32(q_out, (size_t)t * n_heads * hd + h * hd + kk + half, a * ss + b * cc);
        return;
    }
    const float a = k[(size_t)t * ldk + h * hd + kk], b = k[(size_t)t * ldk + h * hd + kk + half];
    const float va = v[(size_t)t * ldv + h * hd + kk], vb = v[(size_t)t * ldv + h * hd + kk + half];
    const int p = pos[t];
    const long page = table[(size_t)slot[t] * table_stride + p / page_size];
    const int place = p % page_size;
    TC* kbase = cache + page * page_stride;
    TC* vbase = kbase + (size_t)n_kv * page_size * hd;
    const size_t o = ((size_t)h * page_size + place) * hd;
    store_f32(kbase, o + kk, a * cc - b * ss);
    store_f32(kbase, o + kk + half, a * ss + b * cc);
    store_f32(vbase, ((size_t)h * hd + kk) * page_size + place, va);
    store_f32(vbase, ((size_t)h * hd + kk + half) * page_size + place, vb);
}

GI_API int gi_rope_store(const float* q, const float* k, const float* v, long ldq, long ldk, long ldv, const float* cos_t,
                         const float* sin_t, const int* pos, const int* slot, const int* table, int table_stride, void* q_out,
                         int q_dtype, void* cache, int cache_dtype, long page_stride, int page_size, int n_rows, int n_heads,
                         int n_kv, int hd, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_heads > 0 && n_kv > 0 && hd > 0 && hd % 2 == 0, "rope_store: bad sizes (rows %d heads %d kv %d hd %d)",
               n_rows, n_heads, n_kv, hd);
    GI_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "rope_store: cos and sin must both be given or both be absent");
    GI_REQUIRE(k == nullptr || (v != nullptr && cache != nullptr && table != nullptr && page_size > 0 &&
                                page_stride >= 2L * n_kv * page_size * hd),
               "rope_store: cache write needs v, a cache, a table and a page stride of at least 2*n_kv*page_size*hd");
    const int items = (n_heads + (k ? n_kv : 0)) * (hd / 2);
    dim3 grid(n_rows, (items + 255) / 256);
    GI_REQUIRE(grid.y <= 65535, "rope_store: too many heads");
#define LAUNCH(TQ, TC)                                                                                                       \
    rope_store_kernel<TQ, TC><<<grid, 256, 0, stream>>>(q, k, v, ldq, ldk, ldv, cos_t, sin_t, pos, slot, table, table_stride, \
                                                          (TQ*)q_out, (TC*)cache, page_stride, page_size, n_heads, n_kv, hd)
    if (q_dtype == GI_F32 && cache_dtype == GI_F32) LAUNCH(float, float);
    else if (q_dtype == GI_BF16 && cache_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t);
    else if (q_dtype == GI_F32 && cache_dtype == GI_BF16) LAUNCH(float, bf16_t);
    else if (q_dtype == GI_BF16 && cache_dtype == GI_F32) LAUNCH(bf16_t, float);
    else return gi_fail("rope_store: unknown dtypes %d, %d", q_dtype, cache_dtype);
#undef LAUNCH
    GI_CHECK_LAUNCH("rope_store");
    return 0;
}

// ------------------------------------------------------------------------------------ SiLU gate
// h[t, i] = silu(gu[t, i]) * gu[t, inter + i], silu(g) = g * (1 / (1 + exp(-g)))
// (src/gpu/device_kernels.inc:460-469).  gu is the product with the stacked [gate; up] matrix.
template <typename TO>
__global__ void silu_mul_kernel(const float* __restrict__ gu, TO* __restrict__ h, int inter, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t t = i / inter, c = i % inter;
    const float g = gu[t * 2 * inter + c], u = gu[t * 2 * inter + inter + c];
    store_f32(h, i, (g * (1.0f / (1.0f + expf(-g)))) * u);
}

GI_API int gi_silu_mul(const float* gate_up, void* h, int h_dtype, int n_rows, int inter, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && inter > 0, "silu_mul: n_rows %d and inter %d must be positive", n_rows, inter);
    const size_t n = (size_t)n_rows * inter;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (h_dtype == GI_F32) silu_mul_kernel<float><<<blocks, 256, 0, stream>>>(gate_up, (float*)h, inter, n);
    else if (h_dtype == GI_BF16) silu_mul_kernel<bf16_t><<<blocks, 256, 0, stream>>>(gate_up, (bf16_t*)h, inter, n);
    else return gi_fail("silu_mul: unknown dtype %d", h_dtype);
    GI_CHECK_LAUNCH("silu_mul");
    return 0;
}

// ----------------------------------------------------------------------------------- row gather
// out[i, :] = x[rows[i], :] (the rows whose logits are wanted; src/gpu/gpu_transformer.cpp:441).
__global__ void gather_rows_kernel(const float* __restrict__ x, const int* __restrict__ rows, float* __restrict__ out, int dim) {
    const float* src = x + (size_t)rows[blockIdx.x] * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) out[(size_t)blockIdx.x * dim + d] = src[d];
}

GI_API int gi_gather_rows(const float* x, const int* rows, float* out, int n_out, int dim, hipStream_t stream) {
    GI_REQUIRE(n_out > 0 && dim > 0, "gather_rows: n_out %d and dim %d must be positive", n_out, dim);
    gather_rows_kernel<<<n_out, 256, 0, stream>>>(x, rows, out, dim);
    GI_CHECK_LAUNCH("gather_rows");
    return 0;
}

// ------------------------------------------------------------------------------- row transforms
// In place over float32 rows [n_rows, dim] with row stride `stride`: x <- x * factor, or x <- cap * tanh(x / cap).
template <bool CAP>
__global__ void rows_in_place_kernel(float* __restrict__ x, int dim, long stride, float c) {
    float* row = x + (size_t)blockIdx.x * stride;
    for (int d = blockIdx.y * blockDim.x + threadIdx.x; d < dim; d += gridDim.y * blockDim.x) row[d] = CAP ? c * tanhf(row[d] / c) : row[d] * c;
}

GI_API int gi_scale_rows(float* x, int n_rows, int dim, long stride, float factor, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0 && stride >= dim, "scale_rows: bad sizes (rows %d, dim %d, stride %ld)", n_rows, dim, stride);
    rows_in_place_kernel<false><<<dim3(n_rows, min(64, (dim + 1023) / 1024)), 256, 0, stream>>>(x, dim, stride, factor);
    GI_CHECK_LAUNCH("scale_rows");
    return 0;
}

GI_API int gi_softcap_rows(float* x, int n_rows, int dim, long stride, float cap, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0 && stride >= dim, "softcap_rows: bad sizes (rows %d, dim %d, stride %ld)", n_rows, dim, stride);
    GI_REQUIRE(cap > 0.f, "softcap_rows: the cap %g must be positive", (double)cap);
    rows_in_place_kernel<true><<<dim3(n_rows, min(64, (dim + 1023) / 1024)), 256, 0, stream>>>(x, dim, stride, cap);
    GI_CHECK_LAUNCH("softcap_rows");
    return 0;
}

// ------------------------------------------------------------------------------- random weights
// out[i] = offset + scale * z_i with z_i a standard normal number that is a function of (key, i) alone, so that a model's random
// weights can be re-made anywhere from the seed and the tensors' names (the key is made of both on the host):
//   r  = mix(key + (i + 1) * 0x9E3779B97F4A7C15)      mix: the splitmix64 finaliser
//   u1 = ((r >> 40) + 1) / 2^24  in (0, 1],  u2 = ((r >> 8) & 0xFFFFFF) / 2^24  in [0, 1)
//   z  = sqrt(-2 ln u1) * cos(2 pi u2)                 in 64-bit; offset + scale * z is rounded to 32-bit, then to the storage type
__device__ __forceinline__ uint64_t splitmix_finish(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

template <typename T>
__global__ __launch_bounds__(256) void random_normal_kernel(T* __restrict__ out, size_t n, uint64_t key, double offset, double scale) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const uint64_t r = splitmix_finish(key + (uint64_t)(i + 1) * 0x9E3779B97F4A7C15ull);
        const double u1 = (double)((r >> 40) + 1) * (1.0 / 16777216.0), u2 = (double)((r >> 8) & 0xFFFFFFull) * (1.0 / 16777216.0);
        const double z = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2);
        store_f32(out, i, (float)(offset + scale * z));
    }
}

GI_API int gi_random_normal(void* out, int dtype, long n, unsigned long long key, double offset, double scale, hipStream_t stream) {
    GI_REQUIRE(out != nullptr && n > 0, "random_normal: bad arguments (n %ld)", n);
    const unsigned grid = (unsigned)min((n + 255) / 256, (long)gi_compute_units() * 16);
    if (dtype == GI_F32) random_normal_kernel<float><<<grid, 256, 0, stream>>>((float*)out, (size_t)n, key, offset, scale);
    else if (dtype == GI_BF16) random_normal_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, (size_t)n, key, offset, scale);
    else return gi_fail("random_normal: unknown dtype %d", dtype);
    GI_CHECK_LAUNCH("random_normal");
    return 0;
}

// --------------------------------------------------------- a norm on a sublayer's output, added on
// x[t, :] += w * (y[t, :] * rsqrt(mean(y[t, :]^2) + eps)): what a "sandwich" layer does with what its mixer or its
// feed-forward puts out.  One workgroup per row; the sum of squares in 32-bit in an order that the row's length fixes.
template <typename TW>
__global__ __launch_bounds__(256) void rmsnorm_add_kernel(const float* __restrict__ y, const TW* __restrict__ w, float* __restrict__ x, int dim,
                                                         float eps, size_t y_stride, size_t x_stride) {
    __shared__ float red[4];
    const float* yr = y + (size_t)blockIdx.x * y_stride;
    float* xr = x + (size_t)blockIdx.x * x_stride;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) ss = fmaf(yr[d], yr[d], ss);
    ss = block_sum<256>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)dim + eps);
    for (int d = threadIdx.x; d < dim; d += 256) xr[d] += load_f32(w, d) * (scale * yr[d]);
}

GI_API int gi_rmsnorm_add(const float* y, const void* w, int w_dtype, float* x, int n_rows, int dim, float eps, long y_stride, long x_stride,
                          hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0 && y_stride >= dim && x_stride >= dim, "rmsnorm_add: bad sizes (rows %d, dim %d)", n_rows, dim);
    if (w_dtype == GI_F32) rmsnorm_add_kernel<float><<<n_rows, 256, 0, stream>>>(y, (const float*)w, x, dim, eps, (size_t)y_stride, (size_t)x_stride);
    else if (w_dtype == GI_BF16) rmsnorm_add_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(y, (const bf16_t*)w, x, dim, eps, (size_t)y_stride, (size_t)x_stride);
    else return gi_fail("rmsnorm_add: unknown dtype %d", w_dtype);
    GI_CHECK_LAUNCH("rmsnorm_add");
    return 0;
}

// ------------------------------------------- head norm, rotation of a head's first channels, cache write
// The general form of rope_store, one wave per (row, head):
//   a query or key head is first divided by its root mean square and multiplied by `q_norm` / `k_norm` [hd] (if given),
//   then the pairs (i, i + rot/2), i < rot/2, of its first `rot` channels are turned by the row's angles
//   (cos, sin: [n_rows, rot/2]; nullptr or rot = 0: no rotation); the other channels pass;
//   queries go to q_out [n_rows, n_heads*hd]; keys to the page's [kv_head][place][hd]; values, of `vd` channels a head,
//   to the page's [kv_head][vd][place] behind all keys.  k == nullptr: another layer's pages are read and none written.
// Before any of that a projection's bias is added (q_bias [n_heads*hd], k_bias [n_kv*hd], v_bias [n_kv*vd], float32; nullptr: none).
// Values may be blended with those another layer made of the same rows: with `v_other` [n_rows, ld_other] and `v_blend` (one
// number on the device), v <- (1 - blend) v + blend v_other is what goes into the page; `v_keep` [n_rows, ld_keep], if given, gets
// this layer's values (with their bias, before any blending) for such a reader.
// `flags`: NRS_NORM_ALL takes the norm over all heads of the projection at once, with weights [heads * hd] ([kv heads * hd]); NRS_NEIGHBOURS turns the pairs (2i, 2i + 1), i < rot/2, instead (angle i for pair i); NRS_UNIT_RMS divides every query and
// key head by its root mean square without weights (q_norm and k_norm must then be absent); NRS_NORM_LAST takes the norm, of
// either form, behind the rotation instead of in front of it.  `v_scale` multiplies the values on their way into the pages (the
// attention's result is linear in them: a layer that weighs its attention's result can weigh the values instead).
constexpr int NRS_MAX_HD = 512;
constexpr int NRS_NEIGHBOURS = 1, NRS_UNIT_RMS = 2, NRS_NORM_LAST = 4, NRS_NORM_ALL = 8;

// For a norm over all heads of a projection at once (NRS_NORM_ALL): r[t] = {1 / sqrt(mean(q_t^2) + eps), the same of k_t}, the rows with
// their biases, one workgroup a row; every head's wave of the kernel below then reads its row's number instead of adding up the
// whole row once more (which at 32 heads of 128 channels tripled that kernel's time).
__global__ __launch_bounds__(256) void rows_rsqrt_kernel(const float* __restrict__ q, long ldq, int nq, const float* __restrict__ q_bias, const float* __restrict__ k, long ldk,
                                                        int nk, const float* __restrict__ k_bias, float eps, float* __restrict__ r) {
    __shared__ float red[4];
    const size_t t = blockIdx.x;
    float ss = 0.f;
    for (int d = threadIdx.x; d < nq; d += 256) {
        const float x = q_bias ? q[t * ldq + d] + q_bias[d] : q[t * ldq + d];
        ss = fmaf(x, x, ss);
    }
    ss = block_sum<256>(ss, red);
    if (threadIdx.x == 0) r[2 * t] = 1.0f / sqrtf(ss / (float)nq + eps);
    if (k == nullptr) return;
    ss = 0.f;
    for (int d = threadIdx.x; d < nk; d += 256) {
        const float x = k_bias ? k[t * ldk + d] + k_bias[d] : k[t * ldk + d];
        ss = fmaf(x, x, ss);
    }
    ss = block_sum<256>(ss, red);
    if (threadIdx.x == 0) r[2 * t + 1] = 1.0f / sqrtf(ss / (float)nk + eps);
}

template <typename TQ, typename TC, typename TW>
__global__ __launch_bounds__(64) void norm_rope_store_kernel(const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
                                                            long ldq, long ldk, long ldv, const TW* __restrict__ q_norm, const TW* __restrict__ k_norm,
                                                            float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot,
                                                            const int* __restrict__ pos, const int* __restrict__ slot, const int* __restrict__ table,
                                                            int table_stride, TQ* __restrict__ q_out, TC* __restrict__ cache, long page_stride,
                                                            int page_size, int n_heads, int n_kv, int hd, int vd,
                                                            const float* __restrict__ q_bias, const float* __restrict__ k_bias,
                                                            const float* __restrict__ v_bias, const float* __restrict__ v_other, long ld_other,
                                                            const float* __restrict__ v_blend, float* __restrict__ v_keep, long ld_keep, int flags,
                                                            float v_scale, const float* __restrict__ rows_r) {
    __shared__ float s[NRS_MAX_HD];
    const int t = blockIdx.x, item = blockIdx.y, lane = threadIdx.x;
    const int p = pos[t];
    if (item >= n_heads + n_kv) {                      // a value head: copied into its page, transposed
        const int h = item - n_heads - n_kv;
        const long page = table[(size_t)slot[t] * table_stride + p / page_size];
        TC* vbase = cache + page * page_stride + (size_t)n_kv * page_size * hd + (size_t)h * vd * page_size + p % page_size;
        const float blend = v_other ? v_blend[0] : 0.f;
        for (int d = lane; d < vd; d += 64) {
            float x = v[(size_t)t * ldv + h * vd + d];
            if (v_bias) x += v_bias[h * vd + d];
            if (v_keep) v_keep[(size_t)t * ld_keep + h * vd + d] = x;
            if (v_other) x = (1.0f - blend) * x + blend * v_other[(size_t)t * ld_other + h * vd + d];
            store_f32(vbase, (size_t)d * page_size, v_scale * x);
        }
        return;
    }
    const bool is_q = item < n_heads;
    const int h = is_q ? item : item - n_heads;
    const float* src = is_q ? q + (size_t)t * ldq + h * hd : k + (size_t)t * ldk + h * hd;
    const float* bias = is_q ? q_bias : k_bias;
    const TW* w = is_q ? q_norm : k_norm;
    float ss = 0.f;
    for (int d = lane; d < hd; d += 64) {
        const float x = bias ? src[d] + bias[h * hd + d] : src[d];
        s[d] = x;
        ss = fmaf(x, x, ss);
    }
    const bool normed = w != nullptr || (flags & NRS_UNIT_RMS), norm_last = normed && (flags & NRS_NORM_LAST);
    const bool whole = normed && (flags & NRS_NORM_ALL);          // one norm over all heads of the projection: the row's number was made beforehand
    if (whole && w != nullptr) w += h * hd;
    const float r = whole ? rows_r[2 * (size_t)t + (is_q ? 0 : 1)] : normed ? 1.0f / sqrtf(wave_sum(ss) / (float)hd + eps) : 1.0f;      // (a rotation keeps the sum of squares: the same number in front of it and behind it)
    if (normed && !norm_last) {
        for (int d = lane; d < hd; d += 64) s[d] = w != nullptr ? load_f32(w, d) * (r * s[d]) : r * s[d];
    }
    __syncthreads();
    const int half = rot / 2;
    const bool turn = cos_t != nullptr && rot > 0, neighbours = flags & NRS_NEIGHBOURS;
    TC* kdst = nullptr;
    TQ* qdst = nullptr;
    if (is_q) qdst = q_out + ((size_t)t * n_heads + h) * hd;
    else {
        const long page = table[(size_t)slot[t] * table_stride + p / page_size];
        kdst = cache + page * page_stride + ((size_t)h * page_size + p % page_size) * hd;
    }
    for (int d = lane; d < hd; d += 64) {
        float out = s[d];
        if (turn && d < rot) {
            if (neighbours) {
                const float c = cos_t[(size_t)t * half + d / 2], sn = sin_t[(size_t)t * half + d / 2];
                out = (d & 1) ? s[d] * c + s[d - 1] * sn : s[d] * c - s[d + 1] * sn;
            } else {
                const int i = d < half ? d : d - half;
                const float c = cos_t[(size_t)t * half + i], sn = sin_t[(size_t)t * half + i];
                out = d < half ? s[d] * c - s[d + half] * sn : s[d] * c + s[d - half] * sn;
            }
        }
        if (norm_last) out = w != nullptr ? load_f32(w, d) * (r * out) : r * out;
        if (is_q) store_f32(qdst, d, out); else store_f32(kdst, d, out);
    }
}

GI_API int gi_norm_rope_store(const float* q, const float* k, const float* v, long ldq, long ldk, long ldv, const void* q_norm, const void* k_norm,
                              int norm_dtype, float eps, const float* cos_t, const float* sin_t, int rot, const int* pos, const int* slot,
                              const int* table, int table_stride, void* q_out, int q_dtype, void* cache, int cache_dtype, long page_stride,
                              int page_size, int n_rows, int n_heads, int n_kv, int hd, int vd, const float* q_bias, const float* k_bias,
                              const float* v_bias, const float* v_other, long ld_other, const float* v_blend, float* v_keep, long ld_keep,
                              int flags, float v_scale, float* rows_r, hipStream_t stream) {
    if (flags & NRS_NORM_ALL) {
        GI_REQUIRE(rows_r != nullptr && !(flags & NRS_UNIT_RMS) && q_norm != nullptr && (k == nullptr || k_norm != nullptr),
                   "norm_rope_store: a norm over whole projections needs its weights and room for two numbers a row");
        rows_rsqrt_kernel<<<n_rows, 256, 0, stream>>>(q, ldq, n_heads * hd, q_bias, k, ldk, n_kv * hd, k_bias, eps, rows_r);
        GI_CHECK_LAUNCH("norm_rope_store (rows)");
    }
    GI_REQUIRE(!(flags & NRS_UNIT_RMS) || (q_norm == nullptr && k_norm == nullptr), "norm_rope_store: heads divided by their root mean square have no norm weights");
    GI_REQUIRE(!(flags & NRS_NEIGHBOURS) || rot % 2 == 0, "norm_rope_store: neighbouring pairs need an even number of turned channels");
    GI_REQUIRE(n_rows > 0 && n_heads > 0 && n_kv > 0 && hd > 0 && hd <= NRS_MAX_HD && vd > 0, "norm_rope_store: bad sizes (rows %d heads %d kv %d hd %d vd %d)",
               n_rows, n_heads, n_kv, hd, vd);
    GI_REQUIRE((v_other == nullptr || (v_blend != nullptr && ld_other >= (long)n_kv * vd)) && (v_keep == nullptr || ld_keep >= (long)n_kv * vd) &&
               ((v_other == nullptr && v_keep == nullptr && v_bias == nullptr && k_bias == nullptr) || k != nullptr),
               "norm_rope_store: blended, kept or biased values need values of this layer's own, the blend's weight and rows of n_kv*vd numbers");
    GI_REQUIRE((cos_t == nullptr) == (sin_t == nullptr) && rot >= 0 && rot % 2 == 0 && rot <= hd, "norm_rope_store: cos and sin go together, and the rotated channels are an even number within the head");
    GI_REQUIRE(k == nullptr || (v != nullptr && cache != nullptr && table != nullptr && page_size > 0 && page_stride >= (long)n_kv * page_size * (hd + vd)),
               "norm_rope_store: a cache write needs v, a cache, a table and a page stride of at least n_kv*page_size*(hd+vd)");
    GI_REQUIRE(n_heads + 2 * n_kv <= 65535, "norm_rope_store: too many heads");
    dim3 grid(n_rows, n_heads + (k ? 2 * n_kv : 0));
#define LAUNCH(TQ, TC, TW)                                                                                                                    \
    norm_rope_store_kernel<TQ, TC, TW><<<grid, 64, 0, stream>>>(q, k, v, ldq, ldk, ldv, (const TW*)q_norm, (const TW*)k_norm, eps, cos_t, sin_t, rot, pos, \
                                                                slot, table, table_stride, (TQ*)q_out, (TC*)cache, page_stride, page_size, n_heads, n_kv, hd, vd, \
                                                                q_bias, k_bias, v_bias, v_other, ld_other, v_blend, v_keep, ld_keep, flags, v_scale, rows_r)
    if (q_dtype == GI_F32 && cache_dtype == GI_F32 && norm_dtype == GI_F32) LAUNCH(float, float, float);
    else if (q_dtype == GI_BF16 && cache_dtype == GI_BF16 && norm_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t, bf16_t);
    else if (q_dtype == GI_BF16 && cache_dtype == GI_BF16 && norm_dtype == GI_F32) LAUNCH(bf16_t, bf16_t, float);
    else return gi_fail("norm_rope_store: dtypes (%d, %d, %d) are not served", q_dtype, cache_dtype, norm_dtype);
#undef LAUNCH
    GI_CHECK_LAUNCH("norm_rope_store");
    return 0;
}

// -------------------------------------------------------------------- gated feed-forward, by activation
// h[t, i] = act(gu[t, i]) * gu[t, inter + i]; act 0: SiLU, 1: the tanh form of GELU,
// 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).
template <typename TO>
__global__ void act_mul_kernel(const float* __restrict__ gu, TO* __restrict__ h, int inter, size_t n, int act, float limit) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t t = i / inter, c = i % inter;
    const float g = gu[t * 2 * inter + c], u = gu[t * 2 * inter + inter + c];
    store_f32(h, i, gated_act(g, u, act, limit));
}

GI_API int gi_act_mul(const float* gate_up, void* h, int h_dtype, int n_rows, int inter, int act, float limit, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && inter > 0 && act >= 0 && act < GI_N_ACTIVATIONS, "act_mul: n_rows %d and inter %d must be positive, the activation one of the known", n_rows, inter);
    const size_t n = (size_t)n_rows * inter;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (h_dtype == GI_F32) act_mul_kernel<float><<<blocks, 256, 0, stream>>>(gate_up, (float*)h, inter, n, act, limit);
    else if (h_dtype == GI_BF16) act_mul_kernel<bf16_t><<<blocks, 256, 0, stream>>>(gate_up, (bf16_t*)h, inter, n, act, limit);
    else return gi_fail("act_mul: unknown dtype %d", h_dtype);
    GI_CHECK_LAUNCH("act_mul");
    return 0;
}

// ------------------------------------------------------------------------- feed-forward without a gate
// h[t, i] = act(x[t, i]) for the two-parameter activation "xielu": with a = softplus(params[0]) and b = 1/2 + softplus(params[1]),
//   z > 0:  a z^2 + z / 2          z <= 0:  b (exp(z) - 1 - z) + z / 2
// (quadratic on the right, bounded below on the left, slope 1/2 on both sides of 0).  params: two float32 numbers on the device.
__device__ __forceinline__ float softplus_f32(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename TO>
__global__ __launch_bounds__(256) void xielu_kernel(const float* __restrict__ x, long ldx, TO* __restrict__ h, long ldh, int inter, const float* __restrict__ params) {
    // one row a workgroup (blockIdx.x) and 1,024 columns of it (blockIdx.y): four neighbouring columns a thread where the row allows
    const float a = softplus_f32(params[0]), b = 0.5f + softplus_f32(params[1]);
    const float* xr = x + (size_t)blockIdx.x * ldx;
    TO* hr = h + (size_t)blockIdx.x * ldh;
    auto act = [&](float z) { return z > 0.f ? fmaf(a * z, z, 0.5f * z) : fmaf(b, expm1f(z) - z, 0.5f * z); };
    const int c0 = blockIdx.y * 1024 + threadIdx.x * 4;
    if (c0 + 3 < inter && (ldx & 3) == 0 && (((uintptr_t)x) & 15) == 0) {
        const float4 z = *reinterpret_cast<const float4*>(xr + c0);
        store_f32(hr, c0, act(z.x));
        store_f32(hr, c0 + 1, act(z.y));
        store_f32(hr, c0 + 2, act(z.z));
        store_f32(hr, c0 + 3, act(z.w));
    } else {
        for (int c = c0; c < min(c0 + 4, inter); ++c) store_f32(hr, c, act(xr[c]));
    }
}

GI_API int gi_xielu(const float* x, long ldx, void* h, int h_dtype, long ldh, int n_rows, int inter, const float* params, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && inter > 0 && ldx >= inter && ldh >= inter && params != nullptr, "xielu: bad sizes (rows %d, columns %d) or no parameters", n_rows, inter);
    GI_REQUIRE((inter + 1023) / 1024 <= 65535, "xielu: rows too long");
    dim3 grid(n_rows, (inter + 1023) / 1024);
    if (h_dtype == GI_F32) xielu_kernel<float><<<grid, 256, 0, stream>>>(x, ldx, (float*)h, ldh, inter, params);
    else if (h_dtype == GI_BF16) xielu_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, ldx, (bf16_t*)h, ldh, inter, params);
    else return gi_fail("xielu: unknown dtype %d", h_dtype);
    GI_CHECK_LAUNCH("xielu");
    return 0;
}

// The same, and on the way the norm that reads the rows next: x += w * norm(y), then out = w_next * norm(x), with out stored as
// the next product reads it.  A thread reads back only what it wrote itself.
template <typename TW, typename TO>
__global__ __launch_bounds__(256) void rmsnorm_add_norm_kernel(const float* __restrict__ y, const TW* __restrict__ w, float* __restrict__ x,
                                                              const TW* __restrict__ w_next, TO* __restrict__ out, int dim, float eps, float eps_next,
                                                              size_t y_stride, size_t x_stride, size_t out_stride) {
    __shared__ float red[4];
    const float* yr = y + (size_t)blockIdx.x * y_stride;
    float* xr = x + (size_t)blockIdx.x * x_stride;
    TO* orow = out + (size_t)blockIdx.x * out_stride;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) ss = fmaf(yr[d], yr[d], ss);
    ss = block_sum<256>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)dim + eps);
    float sx = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) {
        const float v = xr[d] + load_f32(w, d) * (scale * yr[d]);
        xr[d] = v;
        sx = fmaf(v, v, sx);
    }
    sx = block_sum<256>(sx, red);
    const float scale_next = 1.0f / sqrtf(sx / (float)dim + eps_next);
    for (int d = threadIdx.x; d < dim; d += 256) store_f32(orow, d, load_f32(w_next, d) * (scale_next * xr[d]));
}

GI_API int gi_rmsnorm_add_norm(const float* y, const void* w, const void* w_next, int w_dtype, float* x, void* out, int out_dtype, int n_rows, int dim,
                               float eps, float eps_next, long y_stride, long x_stride, long out_stride, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0 && y_stride >= dim && x_stride >= dim && out_stride >= dim, "rmsnorm_add_norm: bad sizes (rows %d, dim %d)", n_rows, dim);
#define LAUNCH(TW, TO)                                                                                                                            \
    rmsnorm_add_norm_kernel<TW, TO><<<n_rows, 256, 0, stream>>>(y, (const TW*)w, x, (const TW*)w_next, (TO*)out, dim, eps, eps_next, (size_t)y_stride, \
                                                                (size_t)x_stride, (size_t)out_stride)
    if (w_dtype == GI_F32 && out_dtype == GI_F32) LAUNCH(float, float);
    else if (w_dtype == GI_F32 && out_dtype == GI_BF16) LAUNCH(float, bf16_t);
    else if (w_dtype == GI_BF16 && out_dtype == GI_F32) LAUNCH(bf16_t, float);
    else if (w_dtype == GI_BF16 && out_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t);
    else return gi_fail("rmsnorm_add_norm: unknown dtypes %d, %d", w_dtype, out_dtype);
#undef LAUNCH
    GI_CHECK_LAUNCH("rmsnorm_add_norm");
    return 0;
}

// ------------------------------------------------- rows laid side by side, weighted sums of rows, a vector added to every row
// out[t] = [a[t]; b[t]] stored as a product reads it (b == nullptr: a alone, which makes it a conversion of rows).
template <typename TO>
__global__ __launch_bounds__(256) void concat_rows_kernel(const float* __restrict__ a, long lda, int wa, const float* __restrict__ b, long ldb, int wb,
                                                         TO* __restrict__ out, long ldo) {
    const size_t t = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c < wa) store_f32(out + t * ldo, c, a[t * lda + c]);
    else if (c < wa + wb) store_f32(out + t * ldo, c, b[t * ldb + (c - wa)]);
}

GI_API int gi_concat_rows(const float* a, long lda, int wa, const float* b, long ldb, int wb, void* out, int out_dtype, long ldo, int n_rows, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && wa > 0 && wb >= 0 && lda >= wa && (b == nullptr ? wb == 0 : ldb >= wb) && ldo >= wa + wb, "concat_rows: bad sizes (rows %d, %d + %d columns)", n_rows, wa, wb);
    dim3 grid(n_rows, (wa + wb + 255) / 256);
    GI_REQUIRE(grid.y <= 65535, "concat_rows: rows too long");
    if (out_dtype == GI_F32) concat_rows_kernel<float><<<grid, 256, 0, stream>>>(a, lda, wa, b, ldb, wb, (float*)out, ldo);
    else if (out_dtype == GI_BF16) concat_rows_kernel<bf16_t><<<grid, 256, 0, stream>>>(a, lda, wa, b, ldb, wb, (bf16_t*)out, ldo);
    else return gi_fail("concat_rows: unknown dtype %d", out_dtype);
    GI_CHECK_LAUNCH("concat_rows");
    return 0;
}

// x[t] += sa * a[t] + sb * b[t]  (b == nullptr: the first term alone); the two terms are added to each other first.
__global__ __launch_bounds__(256) void add_weighted_kernel(float* __restrict__ x, long ldx, const float* __restrict__ a, long lda, float sa,
                                                          const float* __restrict__ b, long ldb, float sb, int dim) {
    const size_t t = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= dim) return;
    float y = sa * a[t * lda + c];
    if (b != nullptr) y = fmaf(sb, b[t * ldb + c], y);
    x[t * ldx + c] += y;
}

GI_API int gi_add_weighted(float* x, long ldx, const float* a, long lda, float sa, const float* b, long ldb, float sb, int n_rows, int dim, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0 && ldx >= dim && lda >= dim && (b == nullptr || ldb >= dim), "add_weighted: bad sizes (rows %d, dim %d)", n_rows, dim);
    dim3 grid(n_rows, (dim + 255) / 256);
    GI_REQUIRE(grid.y <= 65535, "add_weighted: rows too long");
    add_weighted_kernel<<<grid, 256, 0, stream>>>(x, ldx, a, lda, sa, b, ldb, sb, dim);
    GI_CHECK_LAUNCH("add_weighted");
    return 0;
}

// x[t] += v for every row t.
template <typename TV>
__global__ __launch_bounds__(256) void add_vector_kernel(float* __restrict__ x, long ldx, const TV* __restrict__ v, int dim) {
    const size_t t = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c < dim) x[t * ldx + c] += load_f32(v, c);
}

GI_API int gi_add_vector(float* x, long ldx, const void* v, int v_dtype, int n_rows, int dim, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0 && ldx >= dim, "add_vector: bad sizes (rows %d, dim %d)", n_rows, dim);
    dim3 grid(n_rows, (dim + 255) / 256);
    GI_REQUIRE(grid.y <= 65535, "add_vector: rows too long");
    if (v_dtype == GI_F32) add_vector_kernel<float><<<grid, 256, 0, stream>>>(x, ldx, (const float*)v, dim);
    else if (v_dtype == GI_BF16) add_vector_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, ldx, (const bf16_t*)v, dim);
    else return gi_fail("add_vector: unknown dtype %d", v_dtype);
    GI_CHECK_LAUNCH("add_vector");
    return 0;
}

// out[t, c] = act(u[t, c]) * table[tokens[t], first + c]: a gate on columns of the token's own row of a table.  act: 0 SiLU, 1 the tanh
// form of GELU.
template <typename TT, typename TO>
__global__ __launch_bounds__(64) void gate_token_columns_kernel(const float* __restrict__ u, long ldu, const TT* __restrict__ table, long ldt, int first,
                                                               const int* __restrict__ tokens, TO* __restrict__ out, long ldo, int dim, int act) {
    const size_t t = blockIdx.x;
    const TT* row = table + (size_t)tokens[t] * ldt + first;
    for (int c = threadIdx.x; c < dim; c += 64) {
        const float z = u[t * ldu + c];
        const float a = act == 1 ? 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))) : z / (1.0f + expf(-z));
        store_f32(out + t * ldo, c, a * load_f32(row, c));
    }
}

// The same behind a product of a few rows, all in one: out[t, j] = act(W[j] . a[t]) * table[tokens[t], first + j] with a[t] the 32-bit row
// x[t] as a product reads it (rounded to bfloat16 where `round_rows`).  One wave per (row, output): a lane takes eight neighbouring
// columns at a time, the lanes' sums are added by a butterfly.
template <typename TW, typename TT, typename TO>
__global__ __launch_bounds__(256) void gate_token_columns_rows_kernel(const float* __restrict__ x, long ldx, const TW* __restrict__ w, long ldw, int width,
                                                                     const TT* __restrict__ table, long ldt, int first, const int* __restrict__ tokens,
                                                                     TO* __restrict__ out, long ldo, int dim, int act, int round_rows) {
    const size_t t = blockIdx.x;
    const int j = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (j >= dim) return;
    const float* a = x + t * ldx;
    const TW* wj = w + (size_t)j * ldw;
    float s = 0.f;
    const int whole = width & ~7;
#pragma unroll 4
    for (int d = lane * 8; d < whole; d += 512) {
        float wv[8], av[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) wv[i] = load_f32(wj, d + i), av[i] = a[d + i];
#pragma unroll
        for (int i = 0; i < 8; ++i) s = fmaf(wv[i], round_rows ? bf16_to_f32(f32_to_bf16(av[i])) : av[i], s);
    }
    for (int d = whole + lane; d < width; d += 64) s = fmaf(load_f32(wj, d), round_rows ? bf16_to_f32(f32_to_bf16(a[d])) : a[d], s);
    s = wave_sum(s);
    if (lane == 0) {
        const float g = act == 1 ? 0.5f * s * (1.0f + tanhf(0.7978845608028654f * (s + 0.044715f * s * s * s))) : s / (1.0f + expf(-s));
        store_f32(out + t * ldo, j, g * load_f32(table + (size_t)tokens[t] * ldt + first, j));
    }
}

GI_API int gi_gate_token_columns_rows(const float* x, long ldx, const void* w, int w_dtype, long ldw, int width, const void* table, int table_dtype, long ldt, int first,
                                      const int* tokens, void* out, int out_dtype, long ldo, int n_rows, int dim, int act, int round_rows, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0 && width > 0 && ldx >= width && ldw >= width && ldo >= dim && first >= 0 && ldt >= first + dim && (act == 0 || act == 1),
               "gate_token_columns_rows: bad sizes (rows %d, width %d, dim %d, columns from %d of %ld)", n_rows, width, dim, first, ldt);
    dim3 grid(n_rows, (dim + 3) / 4);
    GI_REQUIRE(grid.y <= 65535, "gate_token_columns_rows: too many columns");
#define LAUNCH(TW, TT, TO)                                                                                                                            \
    gate_token_columns_rows_kernel<TW, TT, TO><<<grid, 256, 0, stream>>>(x, ldx, (const TW*)w, ldw, width, (const TT*)table, ldt, first, tokens, (TO*)out, ldo, dim, act, \
                                                                         round_rows)
    if (w_dtype == GI_BF16 && table_dtype == GI_BF16 && out_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t, bf16_t);
    else if (w_dtype == GI_F32 && table_dtype == GI_F32 && out_dtype == GI_F32) LAUNCH(float, float, float);
    else return gi_fail("gate_token_columns_rows: dtypes (%d, %d, %d) are not served", w_dtype, table_dtype, out_dtype);
#undef LAUNCH
    GI_CHECK_LAUNCH("gate_token_columns_rows");
    return 0;
}

GI_API int gi_gate_token_columns(const float* u, long ldu, const void* table, int table_dtype, long ldt, int first, const int* tokens, void* out, int out_dtype,
                                 long ldo, int n_rows, int dim, int act, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0 && ldu >= dim && ldo >= dim && first >= 0 && ldt >= first + dim && (act == 0 || act == 1),
               "gate_token_columns: bad sizes (rows %d, dim %d, columns from %d of %ld)", n_rows, dim, first, ldt);
#define LAUNCH(TT, TO) gate_token_columns_kernel<TT, TO><<<n_rows, 64, 0, stream>>>(u, ldu, (const TT*)table, ldt, first, tokens, (TO*)out, ldo, dim, act)
    if (table_dtype == GI_F32 && out_dtype == GI_F32) LAUNCH(float, float);
    else if (table_dtype == GI_BF16 && out_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t);
    else if (table_dtype == GI_BF16 && out_dtype == GI_F32) LAUNCH(bf16_t, float);
    else if (table_dtype == GI_F32 && out_dtype == GI_BF16) LAUNCH(float, bf16_t);
    else return gi_fail("gate_token_columns: unknown dtypes %d, %d", table_dtype, out_dtype);
#undef LAUNCH
    GI_CHECK_LAUNCH("gate_token_columns");
    return 0;
}
