// The selective scan (a state-space recurrence whose step size and in/out vectors depend on the token), stepped token by token in
// 32-bit.  Per channel c and state n of a request:
//     S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n        y_c = sum_n S[c, n] C_n + D_c x_c
// with A = -exp(A_log) [channels, states], dt_c = softplus(pre_c + bias_c) one per channel and token, B and C [states] one per
// token.  x is the channel's input behind a short causal convolution (taps [channels, taps], the last tap the token's own, a bias)
// and SiLU; the read-out is multiplied by SiLU of a gate z.  Channels never meet, so a wave owns 16 of them for one request of the
// step and walks the request's rows in order; a channel's states lie over four neighbouring lanes (state n with lane n mod 4),
// whose shares of the read-out's sum are added by lane moves in an order that the number of states alone fixes: a request's
// results have the same bits however its rows are cut into steps.  A token's inputs are asked for while the token before it is
// worked on.
//
// State of one request slot, 32-bit: S [channels][states], then the convolution's last taps - 1 inputs [taps - 1][channels].
#include <type_traits>

#include "common.h"

namespace {

constexpr int SSM_MAX_TAPS = 16;

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }
// The same two by the hardware's exp2, log2 and reciprocal (each within a unit or two in the last place of 32 bits), for results
// that leave as bfloat16.
__device__ __forceinline__ float silu_quick(float z) { return z * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z * -1.4426950408889634f)); }
__device__ __forceinline__ float softplus_quick(float z) {
    return z > 20.f ? z : 0.6931471805599453f * __builtin_amdgcn_logf(1.0f + __builtin_amdgcn_exp2f(z * 1.4426950408889634f));
}
// The value of the lane that the quad permutation CTRL names (within groups of four lanes).
template <int CTRL>
__device__ __forceinline__ float quad_moved(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, false));
}

// How many of the rows t-1, t-2, ... (at most `most`) belong to the same request as row t and directly precede it.
__device__ __forceinline__ int rows_before(const int* __restrict__ slot, const int* __restrict__ pos, int t, int most) {
    int n = 0;
    while (n < most && t - n - 1 >= 0 && slot[t - n - 1] == slot[t] && pos[t - n - 1] == pos[t] - n - 1) ++n;
    return n;
}

// Convolution + bias + SiLU of one row's channels.  Rows of the same request in this step are read where they lie; what came before
// the step comes from the request's tail.  `move_tail` (steps of single rows: nobody else reads this request's tail): the thread that
// read a channel's tail also moves it on.
template <typename TO>
__global__ __launch_bounds__(256) void ssm_conv_kernel(const float* __restrict__ pre, long ld, const float* __restrict__ taps, int n_taps,
                                                      const float* __restrict__ bias, float* __restrict__ tail, long tail_stride, int move_tail,
                                                      const int* __restrict__ slot, const int* __restrict__ pos, float* __restrict__ x,
                                                      TO* __restrict__ x_low, int inner) {
    const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= inner) return;
    const int before = rows_before(slot, pos, t, n_taps - 1);
    float* old = tail + (size_t)slot[t] * tail_stride;
    float y = bias[c];
    for (int j = 0; j < n_taps; ++j) {
        const int back = n_taps - 1 - j;                      // rows before t that tap j reads
        const float v = back <= before ? pre[(size_t)(t - back) * ld + c] : old[(size_t)(n_taps - 1 - (back - before)) * inner + c];
        y = fmaf(taps[(size_t)c * n_taps + j], v, y);
    }
    if (move_tail) {
        for (int i = 0; i + 2 < n_taps; ++i) old[(size_t)i * inner + c] = old[(size_t)(i + 1) * inner + c];
        if (n_taps > 1) old[(size_t)(n_taps - 2) * inner + c] = pre[(size_t)t * ld + c];
    }
    y = silu_f(y);
    x[(size_t)t * inner + c] = y;
    if (x_low != nullptr) store_f32(x_low, (size_t)t * inner + c, y);
}

// Behind the convolution: every request's tail becomes the last taps - 1 inputs of (its old tail, its rows of this step).
__global__ __launch_bounds__(256) void ssm_tail_kernel(const float* __restrict__ pre, long ld, int inner, int n_taps, const int* __restrict__ seg_start,
                                                      const int* __restrict__ seg_len, const int* __restrict__ slot, float* __restrict__ tail,
                                                      long tail_stride) {
    const int n = seg_len[blockIdx.x];
    if (n <= 0) return;
    const int t0 = seg_start[blockIdx.x], keep = n_taps - 1;
    float* mine = tail + (size_t)slot[t0] * tail_stride;
    for (int c = blockIdx.y * 256 + threadIdx.x; c < inner; c += 256 * gridDim.y) {
        float held[SSM_MAX_TAPS];
#pragma unroll
        for (int s = 0; s < SSM_MAX_TAPS; ++s) {
            if (s >= keep) break;
            const int e = n - keep + s;                           // row of the step, or (negative) place before it
            held[s] = e >= 0 ? pre[(size_t)(t0 + e) * ld + c] : mine[(size_t)(keep + e) * inner + c];
        }
#pragma unroll
        for (int s = 0; s < SSM_MAX_TAPS; ++s) {
            if (s >= keep) break;
            mine[(size_t)s * inner + c] = held[s];
        }
    }
}

// The recurrence: one wave per (request of the step, 16 channels).  lane = channel * 4 + part; a lane keeps the states part,
// part + 4, ... of its channel (NPL of them at most).  The rows are taken RB at a time: the inputs of the next RB rows are asked
// for, all at once, before the RB rows at hand are stepped through, and what does not depend on the state (step sizes, the gate's
// SiLU) is made for all of them first, so that between two rows only the state's own multiply-add waits for the row before.
// QUICK: exponentials by the hardware's exp2 (the results leave as bfloat16).
template <int RB, int NPL>
struct ScanRows {
    float x[RB], dt[RB], z[RB], B[RB][NPL], C[RB][NPL];
};

// PHASE 0: a workgroup takes a request's rows of the step from the request's state to its state.  Long runs of rows whose results
// leave as bfloat16 are cut into chunks of `chunk_rows` rows instead, which all run at once:
//   PHASE 1  every chunk but a request's last, from a zero state: where the chunk alone takes the state (`ends` [chunks][channels]
//            [states]) and the sum of its step sizes (`sums` [chunks][channels]); nothing else is stored
//   (ssm_carry_kernel: the state every chunk starts from, chunk after chunk: S <- exp(A * sum) S + end, into `ends`)
//   PHASE 2  every chunk from the state it starts from, with the results; a request's last chunk leaves the request's state.
// The sums of a row are taken in another order than from row to row: the results differ by 32-bit rounding.
struct ScanChunk {
    int t0, n_rows, index, last;      // first row, rows, the chunk's number in the step, whether it is its request's last
};
__device__ __forceinline__ bool find_chunk(ScanChunk& ch, int g, const int* __restrict__ seg_start, const int* __restrict__ seg_len, int n_segs, int chunk_rows) {
    ch.index = g;
    for (int s = 0; s < n_segs; ++s) {
        const int rows = seg_len[s], chunks = (rows + chunk_rows - 1) / chunk_rows;
        if (g < chunks) {
            ch.t0 = seg_start[s] + g * chunk_rows;
            ch.n_rows = min(chunk_rows, rows - g * chunk_rows);
            ch.last = g == chunks - 1;
            return true;
        }
        g -= chunks;
    }
    return false;
}

// Steps of single rows take the kernel with RB = 1 (`single_rows`: the host says so; more rows would be right too, only slow).
// FUSED_DT (such steps): the step sizes' product is made here, dt_pre[t, c] = w_dt[c] . low[t, dt_off .. dt_off + dt_rank),
// a channel's four lanes a quarter of the sum each; `dt_pre` is then not read.
template <int NPL, int RB, bool QUICK, int PHASE, bool FUSED_DT, typename TO>
__global__ __launch_bounds__(64) void ssm_scan_kernel(const float* __restrict__ x, const float* __restrict__ dt_pre, long ld_dt, const float* __restrict__ dt_bias,
                                                     const float* __restrict__ bc, long ld_bc, int b_off, int c_off, const float* __restrict__ z, long ld_z,
                                                     const float* __restrict__ a_log, const float* __restrict__ d_skip, const int* __restrict__ seg_start,
                                                     const int* __restrict__ seg_len, const int* __restrict__ row_slot, float* __restrict__ state,
                                                     long state_stride, TO* __restrict__ out, long ldo, int inner, int n_state, int n_segs, int chunk_rows,
                                                     float* __restrict__ ends, float* __restrict__ sums, float out_scale,
                                                     const bf16_t* __restrict__ w_dt, long ld_w, int dt_off, int dt_rank, int dt_vec) {
    ScanChunk ch;
    if (PHASE == 0) {
        ch.t0 = seg_start[blockIdx.x], ch.n_rows = seg_len[blockIdx.x], ch.index = 0, ch.last = 1;
    } else if (!find_chunk(ch, blockIdx.x, seg_start, seg_len, n_segs, chunk_rows) || (PHASE == 1 && ch.last)) {
        return;
    }
    const int n_rows = ch.n_rows;
    if (n_rows <= 0) return;
    const int t0 = ch.t0, lane = threadIdx.x, part = lane & 3;
    const int c = blockIdx.y * 16 + (lane >> 2);
    const bool live = c < inner;
    const int cc = live ? c : inner - 1;                          // (idle lanes walk along on the last channel and store nothing)
    float* mine = state + (size_t)row_slot[t0] * state_stride + (size_t)cc * n_state;
    float* my_end = PHASE == 0 ? nullptr : ends + ((size_t)ch.index * inner + cc) * n_state;
    const float* from = PHASE == 0 ? mine : my_end;
    float S[NPL], A[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const int n = part + 4 * i;
        S[i] = PHASE != 1 && n < n_state ? from[n] : 0.f;
        A[i] = n < n_state ? -expf(a_log[(size_t)cc * n_state + n]) : 0.f;
        if (QUICK) A[i] *= 1.4426950408889634f;
    }
    const float bias = dt_bias[cc], skip = d_skip[cc];
    float dt_sum = 0.f;
    auto ask = [&](ScanRows<RB, NPL>& rows, int r0) {
#pragma unroll
        for (int j = 0; j < RB; ++j) {
            const size_t t = t0 + min(r0 + j, n_rows - 1);          // (rows behind the last ask for the last again)
            rows.x[j] = x[t * inner + cc];
            if (FUSED_DT && r0 + j >= n_rows) {
                rows.dt[j] = 0.f;                                 // (a row behind the last: nothing of it is kept)
            } else if (FUSED_DT) {
                // a lane takes one run of neighbouring columns: in pieces of eight where the rank and the rows' places allow (dt_vec)
                const int per = (dt_rank + 3) / 4, r_lo = min(part * per, dt_rank), r_hi = min(r_lo + per, dt_rank);
                const float* lo = bc + t * ld_bc + dt_off;
                const bf16_t* wr = w_dt + (size_t)cc * ld_w;
                float s = 0.f;
                int r = r_lo;
                if (dt_vec) {
#pragma unroll 4
                    for (; r + 8 <= r_hi; r += 8) {
                        const uint4 w8 = *reinterpret_cast<const uint4*>(wr + r);
                        const float4 a = *reinterpret_cast<const float4*>(lo + r), b = *reinterpret_cast<const float4*>(lo + r + 4);
                        s = fmaf(a.x, __uint_as_float(w8.x << 16), s), s = fmaf(a.y, __uint_as_float(w8.x & 0xffff0000u), s);
                        s = fmaf(a.z, __uint_as_float(w8.y << 16), s), s = fmaf(a.w, __uint_as_float(w8.y & 0xffff0000u), s);
                        s = fmaf(b.x, __uint_as_float(w8.z << 16), s), s = fmaf(b.y, __uint_as_float(w8.z & 0xffff0000u), s);
                        s = fmaf(b.z, __uint_as_float(w8.w << 16), s), s = fmaf(b.w, __uint_as_float(w8.w & 0xffff0000u), s);
                    }
                }
                for (; r < r_hi; ++r) s = fmaf(lo[r], bf16_to_f32(wr[r]), s);
                s += quad_moved<0xB1>(s);
                s += quad_moved<0x4E>(s);
                rows.dt[j] = s;
            } else {
                rows.dt[j] = dt_pre[t * ld_dt + cc];
            }
            if (PHASE != 1) rows.z[j] = z[t * ld_z + cc];
#pragma unroll
            for (int i = 0; i < NPL; ++i) {
                const int n = min(part + 4 * i, n_state - 1);
                rows.B[j][i] = bc[t * ld_bc + b_off + n];
                if (PHASE != 1) rows.C[j][i] = bc[t * ld_bc + c_off + n];
            }
        }
    };
    ScanRows<RB, NPL> now, next;
    ask(now, 0);
    // The RB rows at hand.  What does not depend on the state comes first, for all rows: step sizes, the gate's SiLU, every state's
    // decay and input.  Then the states step from row to row, one multiply-add each, and every row's read-out is summed over the
    // channel's four lanes.  `whole`: all RB rows exist; otherwise the rows behind the last change nothing and are not stored.
    auto step_rows = [&](int r0, auto whole) {
        constexpr bool WHOLE = decltype(whole)::value;
        float y[RB];
#pragma unroll
        for (int j = 0; j < RB; ++j) {
            now.dt[j] = QUICK ? softplus_quick(now.dt[j] + bias) : softplus_f(now.dt[j] + bias);
            if (PHASE != 1) now.z[j] = QUICK ? silu_quick(now.z[j]) : silu_f(now.z[j]);
        }
#pragma unroll
        for (int j = 0; j < RB; ++j) {
            const bool valid = WHOLE || r0 + j < n_rows;
            const float dt = now.dt[j], dx = dt * now.x[j];
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < NPL; ++i) {
                const float decay = QUICK ? __builtin_amdgcn_exp2f(dt * A[i]) : expf(dt * A[i]);
                const float stepped = fmaf(decay, S[i], dx * now.B[j][i]);
                S[i] = valid ? stepped : S[i];
                if (PHASE != 1) acc = part + 4 * i < n_state ? fmaf(S[i], now.C[j][i], acc) : acc;
            }
            if (PHASE == 1) {
                dt_sum += valid ? dt : 0.f;
                continue;
            }
            acc += quad_moved<0xB1>(acc);                          // lanes 1 apart: quad_perm [1, 0, 3, 2]
            acc += quad_moved<0x4E>(acc);                          // lanes 2 apart: quad_perm [2, 3, 0, 1]
            y[j] = fmaf(skip, now.x[j], acc) * now.z[j] * out_scale;
        }
        if (PHASE != 1 && live && part == 0) {
#pragma unroll
            for (int j = 0; j < RB; ++j)
                if (WHOLE || r0 + j < n_rows) store_f32(out, (size_t)(t0 + r0 + j) * ldo + c, y[j]);
        }
    };
    for (int r0 = 0; r0 < n_rows; r0 += RB) {
        const bool more = r0 + RB < n_rows;
        if (more) ask(next, r0 + RB);
        if (r0 + RB <= n_rows) step_rows(r0, std::true_type{});
        else step_rows(r0, std::false_type{});
        if (more) now = next;
    }
    if (PHASE == 1 && live && part == 0) sums[(size_t)ch.index * inner + c] = dt_sum;
    float* to = PHASE == 1 ? my_end : mine;
    if (live && (PHASE != 2 || ch.last)) {
#pragma unroll
        for (int i = 0; i < NPL; ++i) {
            const int n = part + 4 * i;
            if (n < n_state) to[n] = S[i];
        }
    }
}

// Between the two phases: one wave per (request of the step, 16 channels) walks the request's chunks.  `ends` holds where every chunk
// alone takes the state and gets the state the chunk starts from instead.
template <int NPL, bool QUICK>
__global__ __launch_bounds__(64) void ssm_carry_kernel(const float* __restrict__ a_log, const int* __restrict__ seg_start, const int* __restrict__ seg_len,
                                                      const int* __restrict__ row_slot, const float* __restrict__ state, long state_stride, int inner, int n_state,
                                                      int chunk_rows, float* __restrict__ ends, const float* __restrict__ sums) {
    const int rows = seg_len[blockIdx.x];
    if (rows <= 0) return;
    int first = 0;
    for (int s = 0; s < (int)blockIdx.x; ++s) first += (seg_len[s] + chunk_rows - 1) / chunk_rows;
    const int chunks = (rows + chunk_rows - 1) / chunk_rows, lane = threadIdx.x, part = lane & 3;
    const int c = blockIdx.y * 16 + (lane >> 2);
    if (c >= inner) return;
    const float* mine = state + (size_t)row_slot[seg_start[blockIdx.x]] * state_stride + (size_t)c * n_state;
    float S[NPL], A[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const int n = part + 4 * i;
        S[i] = n < n_state ? mine[n] : 0.f;
        A[i] = n < n_state ? -expf(a_log[(size_t)c * n_state + n]) : 0.f;
        if (QUICK) A[i] *= 1.4426950408889634f;
    }
    for (int g = 0; g < chunks; ++g) {
        float* at = ends + ((size_t)(first + g) * inner + c) * n_state;
        const float sum = g + 1 < chunks ? sums[(size_t)(first + g) * inner + c] : 0.f;
#pragma unroll
        for (int i = 0; i < NPL; ++i) {
            const int n = part + 4 * i;
            if (n < n_state) {
                const float end = g + 1 < chunks ? at[n] : 0.f;
                at[n] = S[i];
                const float decay = QUICK ? __builtin_amdgcn_exp2f(sum * A[i]) : expf(sum * A[i]);
                S[i] = fmaf(decay, S[i], end);
            }
        }
    }
}

}  // namespace

GI_API long gi_ssm_state_floats(int inner, int n_state, int n_taps) { return (long)inner * n_state + (long)(n_taps - 1) * inner; }
GI_API int gi_ssm_max_taps() { return SSM_MAX_TAPS; }
GI_API int gi_ssm_max_states() { return 256; }

GI_API int gi_ssm_conv(const float* pre, long ld, const float* taps, int n_taps, const float* bias, float* state, long state_stride, int move_tail,
                       const int* slot, const int* pos, float* x, void* x_low, int low_dtype, int n_rows, int inner, int n_state, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && inner > 0 && n_state > 0 && ld >= inner && n_taps >= 1 && n_taps <= SSM_MAX_TAPS && state_stride >= gi_ssm_state_floats(inner, n_state, n_taps),
               "ssm_conv: bad sizes (rows %d, channels %d, states %d, taps %d)", n_rows, inner, n_state, n_taps);
    float* tail = state + (size_t)inner * n_state;
    dim3 grid(n_rows, (inner + 255) / 256);
    GI_REQUIRE(grid.y <= 65535, "ssm_conv: too many channels");
    if (x_low == nullptr || low_dtype == GI_F32) ssm_conv_kernel<float><<<grid, 256, 0, stream>>>(pre, ld, taps, n_taps, bias, tail, state_stride, move_tail, slot, pos, x, (float*)x_low, inner);
    else if (low_dtype == GI_BF16) ssm_conv_kernel<bf16_t><<<grid, 256, 0, stream>>>(pre, ld, taps, n_taps, bias, tail, state_stride, move_tail, slot, pos, x, (bf16_t*)x_low, inner);
    else return gi_fail("ssm_conv: unknown dtype %d", low_dtype);
    GI_CHECK_LAUNCH("ssm_conv");
    return 0;
}

GI_API int gi_ssm_tail(const float* pre, long ld, int n_taps, const int* seg_start, const int* seg_len, int n_segs, const int* slot, float* state,
                       long state_stride, int inner, int n_state, hipStream_t stream) {
    GI_REQUIRE(n_segs > 0 && inner > 0 && n_state > 0 && ld >= inner && n_taps >= 1 && n_taps <= SSM_MAX_TAPS && state_stride >= gi_ssm_state_floats(inner, n_state, n_taps),
               "ssm_tail: bad sizes (requests %d, channels %d, taps %d)", n_segs, inner, n_taps);
    if (n_taps == 1) return 0;
    dim3 grid(n_segs, min((inner + 255) / 256, 64));
    ssm_tail_kernel<<<grid, 256, 0, stream>>>(pre, ld, inner, n_taps, seg_start, seg_len, slot, state + (size_t)inner * n_state, state_stride);
    GI_CHECK_LAUNCH("ssm_tail");
    return 0;
}

GI_API int gi_ssm_scan(const float* x, const float* dt_pre, long ld_dt, const float* dt_bias, const float* bc, long ld_bc, int b_off, int c_off, const float* z,
                       long ld_z, const float* a_log, const float* d_skip, const int* seg_start, const int* seg_len, int n_segs, const int* row_slot,
                       float* state, long state_stride, void* out, int out_dtype, long ldo, int inner, int n_state, int n_chunks, int chunk_rows, float* ends,
                       float* sums, float out_scale, const void* w_dt, long ld_w, int dt_off, int dt_rank, int single_rows, hipStream_t stream) {
    GI_REQUIRE(n_segs > 0 && inner > 0 && n_state > 0 && n_state <= 256 && (dt_pre == nullptr || ld_dt >= inner) && ld_z >= inner && ldo >= inner && b_off >= 0 && c_off >= 0
               && ld_bc >= b_off + n_state && ld_bc >= c_off + n_state && state_stride >= (long)inner * n_state,
               "ssm_scan: bad sizes (requests %d, channels %d, states %d)", n_segs, inner, n_state);
    dim3 grid(n_segs, (inner + 15) / 16);
    GI_REQUIRE(grid.y <= 65535, "ssm_scan: too many channels");
    // pieces of eight columns of the step sizes' matrix: every lane's run starts at a multiple of eight, in rows that start at multiples of 16 bytes
    const int dt_vec = w_dt != nullptr && ((dt_rank + 3) / 4) % 8 == 0 && ld_w % 8 == 0 && ((uintptr_t)w_dt & 15) == 0 && ld_bc % 4 == 0 && dt_off % 4 == 0
                       && ((uintptr_t)bc & 15) == 0;
    GI_REQUIRE(w_dt == nullptr || (out_dtype == GI_BF16 && n_chunks == 0 && single_rows && dt_rank > 0 && ld_w >= dt_rank && dt_off >= 0 && ld_bc >= dt_off + dt_rank),
               "ssm_scan: the step sizes' product inside the scan needs bfloat16 results, rows not in chunks, and its columns within the rows of B and C");
    GI_REQUIRE(w_dt != nullptr || dt_pre != nullptr, "ssm_scan: step sizes, or the matrix that makes them, are needed");
    GI_REQUIRE(n_chunks == 0 || (n_chunks > 0 && chunk_rows > 0 && ends != nullptr && sums != nullptr && out_dtype == GI_BF16),
               "ssm_scan: rows in chunks need the chunks' scratch memory and results stored as bfloat16");
#define LAUNCH(NPL, RB, QUICK, TO)                                                                                                                            \
    do {                                                                                                                                                      \
        if (n_chunks == 0 && single_rows && !(QUICK && w_dt != nullptr)) {                                                                                    \
            ssm_scan_kernel<NPL, 1, QUICK, 0, false, TO><<<grid, 64, 0, stream>>>(x, dt_pre, ld_dt, dt_bias, bc, ld_bc, b_off, c_off, z, ld_z, a_log, d_skip, seg_start, \
                                                                                  seg_len, row_slot, state, state_stride, (TO*)out, ldo, inner, n_state, n_segs, 0, nullptr, nullptr, out_scale, \
                                                                                  nullptr, 0, 0, 0, 0);                                                        \
        } else if (n_chunks == 0 && QUICK && w_dt != nullptr) {                                                                                               \
            ssm_scan_kernel<NPL, 1, QUICK, 0, QUICK, TO><<<grid, 64, 0, stream>>>(x, dt_pre, ld_dt, dt_bias, bc, ld_bc, b_off, c_off, z, ld_z, a_log, d_skip, seg_start, \
                                                                                   seg_len, row_slot, state, state_stride, (TO*)out, ldo, inner, n_state, n_segs, 0, nullptr, nullptr, out_scale, \
                                                                                   (const bf16_t*)w_dt, ld_w, dt_off, dt_rank, dt_vec);                                \
        } else if (n_chunks == 0) {                                                                                                                           \
            ssm_scan_kernel<NPL, RB, QUICK, 0, false, TO><<<grid, 64, 0, stream>>>(x, dt_pre, ld_dt, dt_bias, bc, ld_bc, b_off, c_off, z, ld_z, a_log, d_skip, seg_start, \
                                                                                   seg_len, row_slot, state, state_stride, (TO*)out, ldo, inner, n_state, n_segs, 0, nullptr, nullptr, out_scale, \
                                                                                   nullptr, 0, 0, 0, 0);                                                        \
        } else {                                                                                                                                              \
            dim3 by_chunk(n_chunks, grid.y);                                                                                                                  \
            ssm_scan_kernel<NPL, (RB > 3 ? RB / 4 : 1), QUICK, 1, false, TO><<<by_chunk, 64, 0, stream>>>(x, dt_pre, ld_dt, dt_bias, bc, ld_bc, b_off, c_off, z, ld_z, a_log, d_skip, seg_start, \
                                                                                seg_len, row_slot, state, state_stride, (TO*)out, ldo, inner, n_state, n_segs, chunk_rows, ends, sums, out_scale, nullptr, 0, 0, 0, 0); \
            ssm_carry_kernel<NPL, QUICK><<<grid, 64, 0, stream>>>(a_log, seg_start, seg_len, row_slot, state, state_stride, inner, n_state, chunk_rows, ends, sums); \
            ssm_scan_kernel<NPL, (RB > 3 ? RB / 4 : 1), QUICK, 2, false, TO><<<by_chunk, 64, 0, stream>>>(x, dt_pre, ld_dt, dt_bias, bc, ld_bc, b_off, c_off, z, ld_z, a_log, d_skip, seg_start, \
                                                                                seg_len, row_slot, state, state_stride, (TO*)out, ldo, inner, n_state, n_segs, chunk_rows, ends, sums, out_scale, nullptr, 0, 0, 0, 0); \
        }                                                                                                                                                     \
    } while (0)
#define BY_STATES(QUICK, TO)                                     \
    do {                                                         \
        if (n_state <= 16) LAUNCH(4, 16, QUICK, TO);             \
        else if (n_state <= 32) LAUNCH(8, 8, QUICK, TO);         \
        else if (n_state <= 64) LAUNCH(16, 4, QUICK, TO);        \
        else if (n_state <= 128) LAUNCH(32, 2, QUICK, TO);       \
        else LAUNCH(64, 1, QUICK, TO);                           \
    } while (0)
    if (out_dtype == GI_F32) BY_STATES(false, float);
    else if (out_dtype == GI_BF16) BY_STATES(true, bf16_t);
    else return gi_fail("ssm_scan: unknown dtype %d", out_dtype);
#undef BY_STATES
#undef LAUNCH
    GI_CHECK_LAUNCH("ssm_scan");
    return 0;
}
