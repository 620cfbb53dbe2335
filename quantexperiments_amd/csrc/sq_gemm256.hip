// Large-tile fp16 GEMM for prefill: Y[T, R] = X[T, C] . W[R, C]^T, fp32 accumulate, optional row scale.
//
// Workgroup tile 256 tokens x 256 weight rows x 64 columns, 4 waves in 2 x 2, each wave a 128 x 128
// tile of sixteen v_mfma_f32_32x32x16_f16 accumulators (256 accumulator registers per lane).  Both
// operands are K-contiguous fp16 in memory; a column tile of each (256 x 64 halves = 32 KB) is copied
// from global memory straight into LDS, double buffered (128 KB), one barrier per column tile.  LDS rows
// are 128 bytes; the 16-byte piece c of row r is stored at slot c ^ ((r >> 1) & 7), which makes the operand
// reads (16 lanes = 16 rows x one piece per cycle) conflict free.
//
// Operand layout of v_mfma_f32_32x32x16_f16, lane l: A row / B column l % 32, k = 8 * (l / 32) .. + 7;
// D[v], v = 0..15: row 8 * (v / 4) + 4 * (l / 32) + v % 4, column l % 32.  Rows of D are tokens, columns
// are weight rows, so a half-wave stores 32 consecutive outputs of one token.
#include "sq_common.h"

namespace sq {

constexpr int G_BM = 256, G_BN = 256, G_BK = 64;

struct Gemm256Args {
    const uint16_t* x;        // fp16 [T, C], row stride ldx
    const uint16_t* w;        // fp16 [R, C], row stride ldw
    const uint16_t* row_scale;  // fp16 [R] or NULL (no scaling)
    void* y;
    int64_t ldx, ldw, ldy;
    int T, R, C, y_off, y_dtype;
    int tiles_t, tiles_r;     // token / weight-row tiles (for the workgroup -> tile mapping)
};

__device__ __forceinline__ int swz(int r, int c) { return c ^ ((r >> 1) & 7); }

__global__ __launch_bounds__(256) void gemm256_kernel(Gemm256Args a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // [2 buffers][X tile 32 KB | W tile 32 KB]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // consecutive tiles walk the token tiles of one weight tile, so a weight tile is fetched from HBM once and
    // its re-reads hit L2 while the (small) activation matrix stays resident
    // Workgroups are dealt round-robin to the 8 XCDs (each with its own L2), so workgroup i of the launch
    // takes tile (i % 8) * (n / 8) + i / 8: every XCD then works on one contiguous run of tiles and a weight
    // tile is fetched by one L2 only.  The grid is padded to a multiple of 8; surplus workgroups leave.
    const int per_xcd = gridDim.x >> 3;
    const int tile = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (tile >= a.tiles_t * a.tiles_r) return;
    const int bt = tile % a.tiles_t, br = tile / a.tiles_t;
    const int t0 = bt * G_BM, r0 = br * G_BN;
    const int wm = (wave >> 1) * 128, wn = (wave & 1) * 128;

    float16v acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // Staging goes straight from global memory into LDS (global_load_lds_dwordx4: no staging registers, no
    // LDS store instructions).  One such load fills 1 KB = 8 LDS rows in lane order, so lane s lands in LDS
    // row s >> 3, slot s & 7 of its chunk, and therefore fetches the piece that the swizzle puts there:
    // piece (s & 7) ^ f(row).  A tile is 32 chunks; wave w fills chunks 8 w .. 8 w + 7 of both operands.
    // Global addresses are a uniform base (advanced per column tile) plus per-lane 32-bit element offsets
    // computed once; rows past the matrix edge re-read the last row (their outputs are never stored).
    const int lrow = lane >> 3, slot = lane & 7;
    uint32_t xo[8], wo[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int row = (wave * 8 + j) * 8 + lrow;
        const int c = slot ^ ((row >> 1) & 7);
        const int t = t0 + row < a.T ? row : a.T - 1 - t0;
        const int r = r0 + row < a.R ? row : a.R - 1 - r0;
        xo[j] = (uint32_t)(t * (int)a.ldx + c * 8);
        wo[j] = (uint32_t)(r * (int)a.ldw + c * 8);
    }
    const uint16_t* xt = a.x + (int64_t)t0 * a.ldx;
    const uint16_t* wt = a.w + (int64_t)r0 * a.ldw;
    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    auto stage = [&](int k0, int buf) {
        const uint16_t* xk = xt + k0;
        const uint16_t* wk = wt + k0;
        unsigned char* dx = smem + buf * 65536 + wave * 8192;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            __builtin_amdgcn_global_load_lds((gptr_t)(xk + xo[j]), (lptr_t)(dx + j * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(wk + wo[j]), (lptr_t)(dx + 32768 + j * 1024), 16, 0, 0);
        }
    };

    // Operand fragments.  The swizzle term depends only on row mod 16 and the rows a lane reads differ by
    // multiples of 32, so one base offset per operand plus compile-time multiples of 32 rows (4096 bytes)
    // covers them all; the column step kk only flips bits 5-6 of the offset (kk << 5).
    half8v fa[4][4], fb[4][4];
    const int frow = lane & 31, fhalf = lane >> 5;
    const uint32_t fa_off = (uint32_t)((wm + frow) * 128 + swz(frow, fhalf) * 16);
    const uint32_t fb_off = (uint32_t)((wn + frow) * 128 + swz(frow, fhalf) * 16 + 32768);
    auto load_frags = [&](const unsigned char* buf, int kk) {
        const unsigned char* pa = buf + (fa_off ^ (uint32_t)(kk << 5));
        const unsigned char* pb = buf + (fb_off ^ (uint32_t)(kk << 5));
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[kk][i] = *reinterpret_cast<const half8v*>(pa + i * 4096);
#pragma unroll
        for (int j = 0; j < 4; ++j) fb[kk][j] = *reinterpret_cast<const half8v*>(pb + j * 4096);
    };
    auto multiply = [&](int kk) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[kk][i], fb[kk][j], acc[i][j], 0, 0, 0);
    };

    // Column-tile loop: read all of this tile's fragments (the matrix instructions start as the first ones
    // arrive), then start the next tile's transfer into the other buffer, then multiply.  No LDS read follows
    // the transfer inside an iteration, so nothing waits for it before the barrier at the end.
    const int nk = a.C / G_BK;
    stage(0, 0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const unsigned char* buf = smem + (kt & 1) * 65536;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) load_frags(buf, kk);
        __builtin_amdgcn_sched_barrier(0);
        if (kt + 1 < nk) stage((kt + 1) * G_BK, (kt + 1) & 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) multiply(kk);
        __syncthreads();
    }

    // epilogue
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int r = r0 + wn + j * 32 + (lane & 31);
        if (r >= a.R) continue;
        const float sc_r = a.row_scale ? h2f(a.row_scale[r]) : 1.f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int t = t0 + wm + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (t >= a.T) continue;
                const float val = acc[i][j][v] * sc_r;
                const int64_t o = (int64_t)t * a.ldy + a.y_off + r;
                if (a.y_dtype == SQ_BF16) reinterpret_cast<uint16_t*>(a.y)[o] = f2bf(val);
                else if (a.y_dtype == SQ_F16) reinterpret_cast<uint16_t*>(a.y)[o] = f2h(val);
                else reinterpret_cast<float*>(a.y)[o] = val;
            }
    }
}

// fp16 copy of a bf16 activation matrix (round to nearest even; exact for every fp16-normal value)
__global__ __launch_bounds__(256) void bf16_to_f16_kernel(const uint16_t* __restrict__ x, int64_t ldx, int T, int C,
                                                          uint16_t* __restrict__ out) {
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;       // 8 elements per thread
    if (i >= (int64_t)T * C) return;
    const int t = (int)(i / C), c = (int)(i - (int64_t)t * C);
    u32x4 v = *reinterpret_cast<const u32x4*>(x + (int64_t)t * ldx + c);
    v.x = bf2h_x2(v.x); v.y = bf2h_x2(v.y); v.z = bf2h_x2(v.z); v.w = bf2h_x2(v.w);
    *reinterpret_cast<u32x4*>(out + i) = v;
}

bool gemm256_ok(int C, int64_t ldx, int64_t ldw, const void* x, const void* w) {
    return C % G_BK == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0;
}

// x and w fp16.  row_scale may be NULL.
int launch_gemm256(const uint16_t* x, int64_t ldx, const uint16_t* w, int64_t ldw, const uint16_t* row_scale, void* y,
                   int y_dtype, int64_t ldy, int y_off, int T, int R, int C, hipStream_t s) {
    static bool raised = false;
    if (!raised) {
        (void)hipFuncSetAttribute((const void*)gemm256_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        (void)hipGetLastError();
        raised = true;
    }
    Gemm256Args a;
    a.x = x; a.w = w; a.row_scale = row_scale; a.y = y; a.ldx = ldx; a.ldw = ldw; a.ldy = ldy;
    a.T = T; a.R = R; a.C = C; a.y_off = y_off; a.y_dtype = y_dtype;
    a.tiles_t = (T + G_BM - 1) / G_BM;
    a.tiles_r = (R + G_BN - 1) / G_BN;
    const unsigned grid = (unsigned)((a.tiles_t * a.tiles_r + 7) / 8 * 8);
    hipLaunchKernelGGL(gemm256_kernel, dim3(grid), dim3(256), 131072, s, a);
    return check_launch("sq_linear_gemm(gemm256)");
}

int launch_bf16_to_f16(const uint16_t* x, int64_t ldx, int T, int C, uint16_t* out, hipStream_t s) {
    const int64_t n = ((int64_t)T * C + 7) / 8;
    hipLaunchKernelGGL(bf16_to_f16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, x, ldx, T, C, out);
    return check_launch("sq_linear_gemm(bf16_to_f16)");
}

}  // namespace sq
