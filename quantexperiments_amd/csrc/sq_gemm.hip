// Prefill product Y[T, R] = X[T, C] . W^T on fp16 MFMA (v_mfma_f32_32x32x16_f16), fp32 accumulate.
//
// The MFMA's B operand wants, per lane, 8 consecutive k of one weight row: exactly one d = 8
// codeword (or two d = 4 codewords), so a weight tile is "dequantised" by gathering raw fp16
// codewords into an LDS tile; the row scale multiplies the fp32 accumulator in the epilogue,
// which keeps the tile exact.  bf16 activations are converted to fp16 while they are staged
// (exact for every fp16-normal value); fp16 MFMA runs at the bf16 rate on gfx950 and keeps the
// codewords' 11-bit significands, which bf16 tiles would cut to 8.
//
// Operand layout of v_mfma_f32_32x32x16_f16 (A: 32 x 16, B: 16 x 32, D: 32 x 32), lane l:
//   A: row l % 32, k = 8 * (l / 32) .. + 7        (tokens)
//   B: col l % 32, k = 8 * (l / 32) .. + 7        (weight rows)
//   D[v], v = 0..15: row 8 * (v / 4) + 4 * (l / 32) + v % 4, col l % 32
#include <algorithm>
#include "sq_common.h"

namespace sq {

constexpr int BM = 128, BN = 128, BK = 32, LDT = BK + 8;   // LDT: padded LDS row stride (halves)

struct GemmArgs {
    sq_matrix m;          // codebook piece (fused) ...
    const uint16_t* wd;   // ... or dense weight [R, C] with row stride ldw (m.R, m.C, m.y_off still valid)
    int64_t ldw;
    const uint16_t* x;
    int64_t ldx;
    void* y;
    int64_t ldy;
    int T;
    int x_dtype, y_dtype, w_dtype;   // w_dtype: element type of wd
};

// 8 consecutive halves of activation row t starting at column k (zeros outside the matrix)
__device__ __forceinline__ u32x4 load_x8(const GemmArgs& a, int t, int k) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (t < a.T && k < a.m.C) {
        v = *reinterpret_cast<const u32x4*>(a.x + (int64_t)t * a.ldx + k);
        if (a.x_dtype == SQ_BF16) { v.x = bf2h_x2(v.x); v.y = bf2h_x2(v.y); v.z = bf2h_x2(v.z); v.w = bf2h_x2(v.w); }
    }
    return v;
}

// 8 consecutive raw weights (unscaled codewords, or dense halves) of row r starting at column k
template <int D, bool DENSE>
__device__ __forceinline__ u32x4 load_w8(const GemmArgs& a, int r, int k) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (r >= a.m.R || k >= a.m.C) return v;
    if (DENSE) {
        v = *reinterpret_cast<const u32x4*>(a.wd + (int64_t)r * a.ldw + k);
        if (a.w_dtype == SQ_BF16) { v.x = bf2h_x2(v.x); v.y = bf2h_x2(v.y); v.z = bf2h_x2(v.z); v.w = bf2h_x2(v.w); }
        return v;
    }
    const sq_matrix& m = a.m;
    const uint32_t* row = reinterpret_cast<const uint32_t*>(m.tags) + (int64_t)r * m.W;
    const uint32_t boff = m.row_book ? (uint32_t)m.row_book[r] << m.bits : 0u;
    if (D == 8) {
        const uint32_t tag = tag_at(row, m.W, m.bits, k >> 3) + boff;
        v = *reinterpret_cast<const u32x4*>(m.table + (size_t)tag * 8);
    } else {
        const uint32_t t0 = tag_at(row, m.W, m.bits, k >> 2) + boff;
        const uint32_t t1 = tag_at(row, m.W, m.bits, (k >> 2) + 1) + boff;
        const u32x2 c0 = *reinterpret_cast<const u32x2*>(m.table + (size_t)t0 * 4);
        const u32x2 c1 = *reinterpret_cast<const u32x2*>(m.table + (size_t)t1 * 4);
        v.x = c0.x; v.y = c0.y; v.z = c1.x; v.w = c1.y;
    }
    return v;
}

template <int D, bool DENSE>
__global__ __launch_bounds__(256) void gemm_kernel(GemmArgs a) {
    __shared__ __attribute__((aligned(16))) uint16_t sx[BM * LDT];
    __shared__ __attribute__((aligned(16))) uint16_t sw[BN * LDT];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t0 = blockIdx.y * BM, r0 = blockIdx.x * BN;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;     // wave tile origin inside the block tile
    float16v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // staging assignment: 512 16-byte pieces per tile, two per thread
    const int sr0 = tid >> 2, sk = (tid & 3) * 8;              // rows sr0 and sr0 + 64, columns sk .. sk + 7
    u32x4 px[2], pw[2];
    px[0] = load_x8(a, t0 + sr0, sk);
    px[1] = load_x8(a, t0 + sr0 + 64, sk);
    pw[0] = load_w8<D, DENSE>(a, r0 + sr0, sk);
    pw[1] = load_w8<D, DENSE>(a, r0 + sr0 + 64, sk);

    for (int k0 = 0; k0 < a.m.C; k0 += BK) {
        __syncthreads();
        *reinterpret_cast<u32x4*>(sx + sr0 * LDT + sk) = px[0];
        *reinterpret_cast<u32x4*>(sx + (sr0 + 64) * LDT + sk) = px[1];
        *reinterpret_cast<u32x4*>(sw + sr0 * LDT + sk) = pw[0];
        *reinterpret_cast<u32x4*>(sw + (sr0 + 64) * LDT + sk) = pw[1];
        __syncthreads();
        if (k0 + BK < a.m.C) {                                  // next tile's loads fly during the MFMAs
            px[0] = load_x8(a, t0 + sr0, k0 + BK + sk);
            px[1] = load_x8(a, t0 + sr0 + 64, k0 + BK + sk);
            pw[0] = load_w8<D, DENSE>(a, r0 + sr0, k0 + BK + sk);
            pw[1] = load_w8<D, DENSE>(a, r0 + sr0 + 64, k0 + BK + sk);
        }
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            half8v fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                fa[i] = *reinterpret_cast<const half8v*>(sx + (wm + i * 32 + (lane & 31)) * LDT + kk + (lane >> 5) * 8);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                fb[j] = *reinterpret_cast<const half8v*>(sw + (wn + j * 32 + (lane & 31)) * LDT + kk + (lane >> 5) * 8);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    }

    // epilogue: row scale on the accumulator, one rounding to the output type
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int r = r0 + wn + j * 32 + (lane & 31);
        if (r >= a.m.R) continue;
        const float sc = a.m.row_scale ? h2f(a.m.row_scale[r]) : 1.f;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int t = t0 + wm + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (t >= a.T) continue;
                const float val = acc[i][j][v] * sc;
                const int64_t o = (int64_t)t * a.ldy + a.m.y_off + r;
                if (a.y_dtype == SQ_BF16) reinterpret_cast<uint16_t*>(a.y)[o] = f2bf(val);
                else if (a.y_dtype == SQ_F16) reinterpret_cast<uint16_t*>(a.y)[o] = f2h(val);
                else reinterpret_cast<float*>(a.y)[o] = val;
            }
    }
}

// ------------------------------------------------------------------------------------------ host

int launch_small_generic(const sq_matrix* mats, int n, const void* x, int x_dtype, int64_t ldx, void* y,
                         int y_dtype, int64_t ldy, int B, hipStream_t s);

bool gemm256_ok(int C, int64_t ldx, int64_t ldw, const void* x, const void* w);
size_t gemm256_part_bytes(int T, int R, int C, int cus);
int launch_gemm256(const uint16_t* x, int64_t ldx, const uint16_t* w, int64_t ldw, const uint16_t* row_scale, void* y,
                   int y_dtype, int64_t ldy, int y_off, int T, int R, int C, float* part, int cus, hipStream_t s);
int launch_bf16_to_f16(const uint16_t* x, int64_t ldx, int T, int C, uint16_t* out, hipStream_t s);
int launch_dequant_with_cvt(const sq_matrix& m, void* out, int64_t ld_out, const uint16_t* x, int64_t ldx, int T, int C,
                            uint16_t* xout, hipStream_t s);

static bool x_vec_ok(const void* x, int64_t ldx, int C) { return C % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x & 15) == 0; }
// Activation rows from which the large-tile route (decode each piece once into the workspace as raw fp16
// codewords, then the 256 x 256 tile GEMM with the row scale in its epilogue) replaces the fused 128 x 128
// kernel, which re-gathers every codeword once per 128 activation rows.  It also wins below 256 rows (7B layer,
// 64 rows: 0.60 ms against 1.90 ms on the fused kernel, whose grid is then a few dozen workgroups), so it is
// used from the first row count sq_linear_small does not take.
constexpr int GEMM256_MIN_T = SQ_SMALL_BMAX + 1;
static size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }
static bool fused_ok(const sq_matrix& m) { return m.tags && (m.d == 8 || m.d == 4) && !m.perms && ((uintptr_t)m.table & 15) == 0; }
static size_t dense_bytes(const sq_matrix& m) { return (((size_t)m.R * m.C * 2) + 255) & ~(size_t)255; }

// The decode + 256 x 256 tile route: from GEMM256_MIN_T rows, and for stacks with column orders at any row count
// (their decode-time kernel is the slow one: 27B-shaped layer with 16 orders, 880 us at 16 rows and 1746 us at 32
// against 625 us here).
static bool big_route(const sq_matrix* mats, int n, int T) {
    if (mats[0].C % 64) return false;
    if (T >= GEMM256_MIN_T) return true;
    for (int i = 0; i < n; ++i)
        if (mats[i].perms) return true;
    return false;
}

// Activation rows from which sq_linear_small hands a stack with column orders to the route above.
constexpr int MASKED_GEMM_FROM = 11;

static bool masked_gemm(const sq_matrix* mats, int n, int B) {
    if (B < MASKED_GEMM_FROM || mats[0].C % 64) return false;
    for (int i = 0; i < n; ++i)
        if (mats[i].perms) return true;
    return false;
}

bool small_takes_gemm_route(const sq_matrix* mats, int n, int B, const void* x, int64_t ldx) {
    return masked_gemm(mats, n, B) && x_vec_ok(x, ldx, mats[0].C);
}

size_t small_gemm_route_workspace(const sq_matrix* mats, int n, int B) {
    return masked_gemm(mats, n, B) ? gemm_workspace(mats, n, B) : 0;
}

// Pieces that are neighbours in Y are decoded one behind the other and multiplied in ONE tile GEMM over all their
// rows (their row scales copied into one array): a 512-row k or v projection alone is 2 tiles of 256 rows, a
// launch that leaves the chip idle (7B q|k|v at 64-255 rows: 139 us as three products, the o projection of q's
// size: 62 us).
constexpr size_t STACK_MAX_BYTES = (size_t)1 << 30;
static bool stacked_route(const sq_matrix* mats, int n) {
    if (n < 2) return false;
    size_t tot = 0;
    for (int i = 0; i < n; ++i) {
        if (mats[i].R <= 0) return false;
        if (i + 1 < n && mats[i + 1].y_off != mats[i].y_off + mats[i].R) return false;
        tot += dense_bytes(mats[i]);
    }
    return tot <= STACK_MAX_BYTES;
}
static int stacked_rows(const sq_matrix* mats, int n) {
    int r = 0;
    for (int i = 0; i < n; ++i) r += mats[i].R;
    return r;
}

__global__ __launch_bounds__(256) void copy_u16_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

static size_t gemm_workspace_beyond_small(const sq_matrix* mats, int n, int T);

size_t gemm_workspace(const sq_matrix* mats, int n, int T) {
    // up to SQ_SMALL_BMAX rows sq_linear_gemm is sq_linear_small, unless the stack goes the other way (see above);
    // which of the two runs then depends on the alignment of x, so the workspace covers both
    if (T > SQ_SMALL_BMAX) return gemm_workspace_beyond_small(mats, n, T);
    const size_t small = small_workspace(mats, n, T);
    return masked_gemm(mats, n, T) ? std::max(small, gemm_workspace_beyond_small(mats, n, T)) : small;
}

static size_t gemm_workspace_beyond_small(const sq_matrix* mats, int n, int T) {
    if (T > SQ_SMALL_BMAX && T <= small_pass_limit(mats, n)) {
        // full passes and the last, shorter one may run different kernels with different needs
        const size_t full = small_workspace(mats, n, SQ_SMALL_BMAX);
        const size_t last = T % SQ_SMALL_BMAX ? small_workspace(mats, n, T % SQ_SMALL_BMAX) : 0;
        return std::max(full, last);
    }
    size_t need = 0;
    const bool big = big_route(mats, n, T);
    if (big && stacked_route(mats, n)) {
        const int R = stacked_rows(mats, n);
        for (int i = 0; i < n; ++i) need += dense_bytes(mats[i]);
        return need + align256((size_t)R * 2) + align256((size_t)T * mats[0].C * 2) + gemm256_part_bytes(T, R, mats[0].C, device_cus());
    }
    for (int i = 0; i < n; ++i)
        if ((big || !fused_ok(mats[i])) && dense_bytes(mats[i]) > need) need = dense_bytes(mats[i]);
    if (big) {
        need += align256((size_t)T * mats[0].C * 2);            // fp16 copy of bf16 activations
        size_t part = 0;                                        // fp32 partial products of a K split
        for (int i = 0; i < n; ++i) part = std::max(part, gemm256_part_bytes(T, mats[i].R, mats[i].C, device_cus()));
        need += part;
    }
    return need;
}

static int run(const GemmArgs& a, int d, bool dense, hipStream_t s) {
    const dim3 grid((a.m.R + BN - 1) / BN, (a.T + BM - 1) / BM);
    if (dense) hipLaunchKernelGGL((gemm_kernel<8, true>), grid, dim3(256), 0, s, a);
    else if (d == 8) hipLaunchKernelGGL((gemm_kernel<8, false>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((gemm_kernel<4, false>), grid, dim3(256), 0, s, a);
    return check_launch("sq_linear_gemm");
}

size_t gemm_dense_workspace(int R, int C, int T) {
    return (T >= GEMM256_MIN_T && C % 64 == 0) ? gemm256_part_bytes(T, R, C, device_cus()) : 0;
}

int launch_gemm_dense(const void* w, int w_dtype, int64_t ldw, int R, int C, const void* x, int x_dtype, int64_t ldx,
                      void* y, int y_dtype, int64_t ldy, int T, hipStream_t s, void* ws, size_t ws_bytes) {
    if (!x_vec_ok(x, ldx, C) || !x_vec_ok(w, ldw, C))
        return fail(SQ_EUNSUPPORTED, "sq_gemm_dense: C, ldx, ldw must be multiples of 8 and pointers 16-byte aligned");
    if (x_dtype == SQ_F16 && w_dtype == SQ_F16 && T >= GEMM256_MIN_T && gemm256_ok(C, ldx, ldw, x, w)) {
        const size_t part = gemm256_part_bytes(T, R, C, device_cus());
        const bool split = ws && part && ws_bytes >= part;
        return launch_gemm256((const uint16_t*)x, ldx, (const uint16_t*)w, ldw, nullptr, y, y_dtype, ldy, 0, T, R, C,
                              split ? (float*)ws : nullptr, split ? device_cus() : 0, s);
    }
    GemmArgs a{};
    a.m.R = R; a.m.C = C; a.m.y_off = 0;
    a.wd = (const uint16_t*)w; a.ldw = ldw;
    a.x = (const uint16_t*)x; a.ldx = ldx; a.y = y; a.ldy = ldy; a.T = T; a.x_dtype = x_dtype; a.y_dtype = y_dtype;
    a.w_dtype = w_dtype;
    return run(a, 8, true, s);
}

int launch_gemm(const sq_matrix* mats, int n, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                int64_t ldy, int T, void* ws, size_t ws_bytes, void* sums, hipStream_t s) {
    if (T <= SQ_SMALL_BMAX && !small_takes_gemm_route(mats, n, T, x, ldx))
        return launch_small(mats, n, x, x_dtype, ldx, y, y_dtype, ldy, T, ws, ws_bytes, sums, s);
    if (T > SQ_SMALL_BMAX && T <= small_pass_limit(mats, n) && x_vec_ok(x, ldx, mats[0].C)) {
        // a few passes of the decode-time kernel read the packed tags a few times; decoding to fp16 first
        // (below) writes and reads 8 to 16 times as many bytes once
        const size_t ys = y_dtype == SQ_F32 ? 4 : 2;
        for (int t = 0; t < T; t += SQ_SMALL_BMAX) {
            const int nb = T - t < SQ_SMALL_BMAX ? T - t : SQ_SMALL_BMAX;
            int rc = launch_small(mats, n, (const char*)x + (size_t)t * ldx * 2, x_dtype, ldx, (char*)y + (size_t)t * ldy * ys,
                                  y_dtype, ldy, nb, ws, ws_bytes, sums, s);
            if (rc) return rc;
        }
        return SQ_OK;
    }
    if (!x_vec_ok(x, ldx, mats[0].C)) {
        for (int i = 0; i < n; ++i)
            if (!mats[i].tags) return fail(SQ_EUNSUPPORTED, "sq_linear_gemm: a matrix held as its tag stream only needs 16-byte aligned x with ldx %% 8 == 0");
        // odd strides: the any-shape kernel, SQ_SMALL_BMAX activation rows at a time
        for (int t = 0; t < T; t += SQ_SMALL_BMAX) {
            const int nb = T - t < SQ_SMALL_BMAX ? T - t : SQ_SMALL_BMAX;
            const size_t es = 2, ys = y_dtype == SQ_F32 ? 4 : 2;
            int rc = launch_small_generic(mats, n, (const char*)x + (size_t)t * ldx * es, x_dtype, ldx,
                                          (char*)y + (size_t)t * ldy * ys, y_dtype, ldy, nb, s);
            if (rc) return rc;
        }
        return SQ_OK;
    }
    if (gemm_workspace(mats, n, T) > ws_bytes)
        return fail(SQ_EWORKSPACE, "sq_linear_gemm: workspace %zu < %zu", ws_bytes, gemm_workspace(mats, n, T));
    if (big_route(mats, n, T)) {
        const int C = mats[0].C;
        const uint16_t* xh = (const uint16_t*)x;
        int64_t ldxh = ldx;
        char* wd = (char*)ws;
        // bf16 activations are copied to fp16 once; the copy rides along with the first decode when that takes
        // the four-chunk kernel (the two overlap in one launch), else it is a launch of its own
        bool copy_pending = x_dtype == SQ_BF16;
        if (copy_pending) {
            xh = (const uint16_t*)ws;
            ldxh = C;
        }
        auto decode = [&](const sq_matrix& m, void* w) -> int {
            if (copy_pending) {
                copy_pending = false;
                const int rc = launch_dequant_with_cvt(m, w, C, (const uint16_t*)x, ldx, T, C, (uint16_t*)ws, s);
                if (rc <= 0) return rc;
                const int rc2 = launch_bf16_to_f16((const uint16_t*)x, ldx, T, C, (uint16_t*)ws, s);
                if (rc2) return rc2;
            }
            return launch_dequant(m, w, SQ_F16, C, 0, m.R, s, /*raw=*/true);
        };
        wd += align256((size_t)T * C * 2);
        const int cus0 = device_cus();
        if (stacked_route(mats, n)) {
            const int R = stacked_rows(mats, n);
            char* next = wd;
            for (int i = 0; i < n; ++i) next += dense_bytes(mats[i]);
            uint16_t* scales = (uint16_t*)next;
            float* part = (float*)(next + align256((size_t)R * 2));
            char* w = wd;
            int r0 = 0;
            for (int i = 0; i < n; ++i) {
                const sq_matrix& m = mats[i];
                int rc = decode(m, w);
                if (rc) return rc;
                hipLaunchKernelGGL(copy_u16_kernel, dim3((unsigned)((m.R + 255) / 256)), dim3(256), 0, s, m.row_scale, scales + r0, m.R);
                rc = check_launch("sq_linear_gemm(row scales)");
                if (rc) return rc;
                w += (size_t)m.R * C * 2;                       // rows follow each other without gaps
                r0 += m.R;
            }
            return launch_gemm256(xh, ldxh, (const uint16_t*)wd, C, scales, y, y_dtype, ldy, mats[0].y_off, T, R, C,
                                  gemm256_part_bytes(T, R, C, cus0) ? part : nullptr, cus0, s);
        }
        size_t dense = 0;
        for (int i = 0; i < n; ++i) dense = std::max(dense, dense_bytes(mats[i]));
        float* part = (float*)(wd + dense);
        const int cus = device_cus();
        for (int i = 0; i < n; ++i) {
            const sq_matrix& m = mats[i];
            if (m.R == 0) continue;
            int rc = decode(m, wd);
            if (rc) return rc;
            rc = launch_gemm256(xh, ldxh, (const uint16_t*)wd, C, m.row_scale, y, y_dtype, ldy, m.y_off, T, m.R, C,
                                gemm256_part_bytes(T, m.R, C, cus) ? part : nullptr, cus, s);
            if (rc) return rc;
        }
        return SQ_OK;
    }
    for (int i = 0; i < n; ++i) {
        const sq_matrix& m = mats[i];
        if (m.R == 0) continue;
        GemmArgs a{};
        a.m = m;
        a.x = (const uint16_t*)x; a.ldx = ldx; a.y = y; a.ldy = ldy; a.T = T; a.x_dtype = x_dtype; a.y_dtype = y_dtype;
        int rc;
        if (fused_ok(m)) {
            rc = run(a, m.d, false, s);
        } else {
            // column orders or an unusual chunk width: gather the raw codewords (with the column
            // scatter) into the workspace as fp16, which is exact, and multiply from there with the row scale
            // applied to the accumulator as in the fused kernel; the stream orders the two kernels and the next piece
            rc = launch_dequant(m, ws, SQ_F16, m.C, 0, m.R, s, /*raw=*/true);
            if (rc) return rc;
            a.wd = (const uint16_t*)ws; a.ldw = m.C; a.w_dtype = SQ_F16;
            rc = run(a, 8, true, s);
        }
        if (rc) return rc;
    }
    return SQ_OK;
}

// ---- the 8-bit block-32 head above SQ_SMALL_BMAX activation rows: row chunks decoded to fp16 (scale folded
// in, one rounding, as the reference's chunked route does: shapequant/vllm_ext/core.py:548-555, 587-591) and
// multiplied by the dense tile GEMM.  A chunk is as large as Q8_CHUNK_BYTES of fp16 allows so that one GEMM
// launch has enough tiles for the whole chip.
constexpr size_t Q8_CHUNK_BYTES = (size_t)256 << 20;

static int q8_chunk_rows(int V, int C) {
    int64_t rows = (int64_t)(Q8_CHUNK_BYTES / ((size_t)C * 2)) / 256 * 256;
    if (rows < 256) rows = 256;
    return rows < V ? (int)rows : V;
}

static bool q8_big(int T, int C) { return T >= GEMM256_MIN_T && C % 64 == 0; }

size_t q8_workspace(int V, int C, int T) {
    if (T <= SQ_SMALL_BMAX || V <= 0) return 0;
    const int chunk = q8_chunk_rows(V, C);
    size_t need = align256((size_t)chunk * C * 2);
    if (q8_big(T, C)) {
        const int last = V % chunk;                             // the split of a launch depends on its tile count
        const size_t part = std::max(gemm256_part_bytes(T, chunk, C, device_cus()),
                                     last ? gemm256_part_bytes(T, last, C, device_cus()) : (size_t)0);
        need += align256((size_t)T * C * 2) + part;
    }
    return need;
}

int launch_q8_large(const int8_t* q, const uint16_t* sc, int V, int C, const void* x, int x_dtype, int64_t ldx, void* y,
                    int y_dtype, int64_t ldy, int T, void* ws, size_t ws_bytes, hipStream_t s) {
    if (q8_workspace(V, C, T) > ws_bytes)
        return fail(SQ_EWORKSPACE, "sq_q8_linear: workspace %zu < %zu", ws_bytes, q8_workspace(V, C, T));
    if (!x_vec_ok(x, ldx, C))
        return fail(SQ_EUNSUPPORTED, "sq_q8_linear: more than %d rows need ldx %% 8 == 0 and 16-byte aligned x", SQ_SMALL_BMAX);
    const int chunk = q8_chunk_rows(V, C);
    const size_t ys = y_dtype == SQ_F32 ? 4 : 2;
    char* wd = (char*)ws;
    const bool big = q8_big(T, C);
    const uint16_t* xh = (const uint16_t*)x;
    int64_t ldxh = ldx;
    float* part = nullptr;
    const int cus = device_cus();
    if (big) {
        if (x_dtype == SQ_BF16) {
            int rc = launch_bf16_to_f16((const uint16_t*)x, ldx, T, C, (uint16_t*)ws, s);
            if (rc) return rc;
            xh = (const uint16_t*)ws;
            ldxh = C;
        }
        wd += align256((size_t)T * C * 2);
        part = (float*)(wd + align256((size_t)chunk * C * 2));
    }
    for (int r0 = 0; r0 < V; r0 += chunk) {
        const int r1 = r0 + chunk < V ? r0 + chunk : V;
        int rc = launch_q8_dequant(q, sc, C, wd, SQ_F16, C, r0, r1, s);
        if (rc) return rc;
        void* yc = (char*)y + (size_t)r0 * ys;
        if (big && gemm256_ok(C, ldxh, C, xh, wd))
            rc = launch_gemm256(xh, ldxh, (const uint16_t*)wd, C, nullptr, yc, y_dtype, ldy, 0, T, r1 - r0, C,
                                gemm256_part_bytes(T, r1 - r0, C, cus) ? part : nullptr, cus, s);
        else
            rc = launch_gemm_dense(wd, SQ_F16, C, r1 - r0, C, x, x_dtype, ldx, yc, y_dtype, ldy, T, s);
        if (rc) return rc;
    }
    return SQ_OK;
}

}  // namespace sq
