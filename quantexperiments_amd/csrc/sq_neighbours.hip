// The two elementwise neighbours of the decode-time products: residual add + RMS norm (writes the next product's
// input) and SiLU(gate) * up (writes the down projection's input), each optionally as M column-order copies.
// They follow addnorm_perm / silu_mul_perm of the reference's decode engine (shapequant/kernels/decode_e2e.py:84-140)
// and the EPI 1 / EPI 2 epilogues of its batch-1 kernel (shapequant/kernels/proto_runs.py:223-287): same arithmetic,
// same rounding points.  Rows are a few thousand elements, so both kernels are latency-bound: one pass over the row
// per workgroup, 16-bit traffic, no workspace.
#include "sq_common.h"

namespace sq {

constexpr int NB_THREADS = 1024;
constexpr int NB_MAX_LDS_C = 32256;          // a row staged as 16-bit values for the column-order copies: 63 KB of LDS

// sum over the workgroup, the same value in every thread
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];                   // same order in every thread
    __syncthreads();
    return t;
}

struct AddnormArgs {
    const float* h_in;
    float* h_out;
    const void* add;
    const void* w;
    const int32_t* perms;
    void* out;
    int64_t ld_h, ld_add;
    int add_dtype, w_dtype, out_dtype, M, C, blocks_per_row, vec;
    float eps;
};

// grid = B * blocks_per_row.  Every workgroup of a row recomputes the norm (the row is small) and writes its share
// of the M copies; the first one writes h_out.  Without column orders there is one workgroup per row, which writes
// element i of h_out after its last read of element i of h_in, so h_out may be h_in then.
__global__ __launch_bounds__(NB_THREADS) void addnorm_kernel(AddnormArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint16_t row16[];
    __shared__ float red[NB_THREADS / 64];
    const int b = blockIdx.x / a.blocks_per_row, part = blockIdx.x % a.blocks_per_row;
    const float* h = a.h_in + (int64_t)b * a.ld_h;
    const int64_t ab = (int64_t)b * a.ld_add;
    uint16_t* out = reinterpret_cast<uint16_t*>(a.out);
    // Mean square in one fixed order (the product kernels that compute this row themselves use the same one, so
    // both give the same bits): slot j of 1024 adds the squares of chunks j, j + 1024, ... (a chunk = 8 consecutive
    // elements, the last one may be short) element by element with fused multiply-adds; each block of 64 slots is
    // folded by the wave butterfly and the 16 block sums are added in turn.
    const int U = (a.C + 7) / 8, tid = threadIdx.x;
    float ss = 0.f;
    if (a.vec && U <= NB_THREADS) {
        // one chunk per thread: 16-byte loads, all in flight at once, values kept for the second half
        float v[8];
        u32x4 wv = u32x4{0u, 0u, 0u, 0u};
        const int c = tid;
        if (c < U) {
            const float4v h0 = reinterpret_cast<const float4v*>(h)[2 * c], h1 = reinterpret_cast<const float4v*>(h)[2 * c + 1];
            wv = reinterpret_cast<const u32x4*>(a.w)[c];
            u32x4 ad = u32x4{0u, 0u, 0u, 0u};
            if (a.add) ad = reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(a.add) + ab)[c];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                v[e] = e < 4 ? h0[e & 3] : h1[e & 3];
                const uint16_t bits = (uint16_t)(ad[e >> 1] >> (16 * (e & 1)));
                if (a.add) v[e] += a.add_dtype == SQ_BF16 ? bf2f(bits) : h2f(bits);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) ss = __builtin_fmaf(v[e], v[e], ss);
        }
        const float rstd = rsqrtf(block_sum(ss, red) / (float)a.C + a.eps);
        if (c < U) {
            u32x4 o;
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                const float w0 = a.w_dtype == SQ_BF16 ? bf2f((uint16_t)wv[e >> 1]) : h2f((uint16_t)wv[e >> 1]);
                const float w1 = a.w_dtype == SQ_BF16 ? bf2f((uint16_t)(wv[e >> 1] >> 16)) : h2f((uint16_t)(wv[e >> 1] >> 16));
                o[e >> 1] = (uint32_t)round16(v[e] * rstd * w0, a.out_dtype) | ((uint32_t)round16(v[e + 1] * rstd * w1, a.out_dtype) << 16);
            }
            if (part == 0 && a.h_out) {
                float4v o0, o1;
#pragma unroll
                for (int e = 0; e < 4; ++e) { o0[e] = v[e]; o1[e] = v[4 + e]; }
                reinterpret_cast<float4v*>(a.h_out + (int64_t)b * a.ld_h)[2 * c] = o0;
                reinterpret_cast<float4v*>(a.h_out + (int64_t)b * a.ld_h)[2 * c + 1] = o1;
            }
            if (a.perms) reinterpret_cast<u32x4*>(row16)[c] = o;
            else reinterpret_cast<u32x4*>(out + (int64_t)b * a.C)[c] = o;
        }
    } else {
        for (int c = tid; c < U; c += NB_THREADS)
            for (int i = c * 8; i < min(c * 8 + 8, a.C); ++i) {
                float v = h[i];
                if (a.add) v += load16(a.add, a.add_dtype, ab + i);
                ss = __builtin_fmaf(v, v, ss);
            }
        const float rstd = rsqrtf(block_sum(ss, red) / (float)a.C + a.eps);
        for (int i = tid; i < a.C; i += NB_THREADS) {
            float v = h[i];
            if (a.add) v += load16(a.add, a.add_dtype, ab + i);
            if (part == 0 && a.h_out) a.h_out[(int64_t)b * a.ld_h + i] = v;
            const uint16_t o = round16(v * rstd * load16(a.w, a.w_dtype, i), a.out_dtype);
            if (a.perms) row16[i] = o;
            else out[(int64_t)b * a.C + i] = o;
        }
    }
    if (!a.perms) return;
    __syncthreads();
    const int n = a.M * a.C;
    for (int k = part * NB_THREADS + threadIdx.x; k < n; k += a.blocks_per_row * NB_THREADS)
        out[(int64_t)b * n + k] = row16[a.perms[k]];
}

struct SiluArgs {
    const void* gate;
    const void* up;
    const int32_t* perms;
    void* out;
    int64_t ld;
    int dtype, M, C, blocks_per_row, vec;
};

__global__ __launch_bounds__(NB_THREADS) void silu_mul_kernel(SiluArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint16_t row16[];
    const int b = blockIdx.x / a.blocks_per_row, part = blockIdx.x % a.blocks_per_row;
    const uint16_t* g = reinterpret_cast<const uint16_t*>(a.gate) + (int64_t)b * a.ld;
    const uint16_t* u = reinterpret_cast<const uint16_t*>(a.up) + (int64_t)b * a.ld;
    uint16_t* out = reinterpret_cast<uint16_t*>(a.out);
    if (!a.perms) {
        if (a.vec) {                                            // 8 elements per thread, 16-byte loads and stores
            for (int c = part * NB_THREADS + threadIdx.x; c < a.C / 8; c += a.blocks_per_row * NB_THREADS) {
                const u32x4 gv = reinterpret_cast<const u32x4*>(g)[c], uv = reinterpret_cast<const u32x4*>(u)[c];
                u32x4 o;
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    o[k] = (uint32_t)silu_mul_one((uint16_t)gv[k], (uint16_t)uv[k], a.dtype) |
                           ((uint32_t)silu_mul_one((uint16_t)(gv[k] >> 16), (uint16_t)(uv[k] >> 16), a.dtype) << 16);
                reinterpret_cast<u32x4*>(out + (int64_t)b * a.C)[c] = o;
            }
            return;
        }
        for (int i = part * NB_THREADS + threadIdx.x; i < a.C; i += a.blocks_per_row * NB_THREADS)
            out[(int64_t)b * a.C + i] = silu_mul_one(g[i], u[i], a.dtype);
        return;
    }
    for (int i = threadIdx.x; i < a.C; i += NB_THREADS) row16[i] = silu_mul_one(g[i], u[i], a.dtype);
    __syncthreads();
    const int n = a.M * a.C;
    for (int k = part * NB_THREADS + threadIdx.x; k < n; k += a.blocks_per_row * NB_THREADS)
        out[(int64_t)b * n + k] = row16[a.perms[k]];
}

// workgroups per activation row: one per 4096 outputs, at most 64 (the copies of a 16-order 18,944-column row are
// 303 K values; one workgroup would take tens of microseconds over them)
static int blocks_for(int64_t outputs) {
    const int64_t n = (outputs + 4095) / 4096;
    return n < 1 ? 1 : n > 64 ? 64 : (int)n;
}

int launch_addnorm(const float* h_in, float* h_out, int64_t ld_h, const void* add, int add_dtype, int64_t ld_add, const void* w,
                   int w_dtype, const int32_t* perms, int M, int B, int C, float eps, void* out, int out_dtype, hipStream_t s) {
    if (perms && C > NB_MAX_LDS_C) return fail(SQ_EUNSUPPORTED, "sq_addnorm: column orders need C <= %d", NB_MAX_LDS_C);
    AddnormArgs a;
    a.h_in = h_in; a.h_out = h_out; a.add = add; a.w = w; a.perms = perms; a.out = out; a.ld_h = ld_h; a.ld_add = ld_add;
    a.add_dtype = add_dtype; a.w_dtype = w_dtype; a.out_dtype = out_dtype; a.M = perms ? M : 1; a.C = C; a.eps = eps;
    a.blocks_per_row = perms ? blocks_for((int64_t)M * C) : 1;
    // 16-byte accesses: whole chunks, every row of every tensor 16-byte aligned
    a.vec = C % 8 == 0 && (B == 1 || (ld_h % 4 == 0 && (!add || ld_add % 8 == 0))) &&
            ((((uintptr_t)h_in | (uintptr_t)h_out | (uintptr_t)add | (uintptr_t)w | (uintptr_t)out) & 15) == 0);
    hipLaunchKernelGGL(addnorm_kernel, dim3((unsigned)(B * a.blocks_per_row)), dim3(NB_THREADS), perms ? (size_t)C * 2 : 0, s, a);
    return check_launch("sq_addnorm");
}

int launch_silu_mul(const void* gate, const void* up, int dtype, int64_t ld, const int32_t* perms, int M, int B, int C, void* out,
                    hipStream_t s) {
    if (perms && C > NB_MAX_LDS_C) return fail(SQ_EUNSUPPORTED, "sq_silu_mul: column orders need C <= %d", NB_MAX_LDS_C);
    SiluArgs a;
    a.gate = gate; a.up = up; a.perms = perms; a.out = out; a.ld = ld; a.dtype = dtype; a.M = perms ? M : 1; a.C = C;
    a.vec = !perms && C % 8 == 0 && ld % 8 == 0 && ((((uintptr_t)gate | (uintptr_t)up | (uintptr_t)out) & 15) == 0);
    a.blocks_per_row = a.vec ? blocks_for((int64_t)C / 2) : blocks_for((int64_t)a.M * C);     // vec: one per 8192 elements
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)(B * a.blocks_per_row)), dim3(NB_THREADS), perms ? (size_t)C * 2 : 0, s, a);
    return check_launch("sq_silu_mul");
}

}  // namespace sq
