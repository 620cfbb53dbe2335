// Large-tile fp16 GEMM for prefill: Y[T, R] = X[T, C] . W[R, C]^T, fp32 accumulate, optional row scale.
//
// Workgroup tile 256 tokens x 256 weight rows, 8 waves in 2 x 4, each wave a 128 x 64 tile of eight
// v_mfma_f32_32x32x16_f16 accumulators (128 accumulator registers per lane), so two waves share a SIMD and
// one issues matrix instructions while the other waits at a barrier.  Both operands are K-contiguous fp16 in
// memory.  The K loop moves in slabs of 64 columns; a slab of ONE operand (256 rows x 128 bytes = 32 KB, whole
// 128-byte lines: half-line requests get 10.5 TB/s out of L2 over the chip, whole lines 15.2 TB/s, and a
// 256 x 256 tile needs about 10 TB/s at the clock the matrix cores sustain) is copied from global memory
// straight into LDS (global_load_lds_dwordx4: no staging registers) into a ring of five 32 KB slots: X_s, W_s,
// X_s+1, W_s+1, X_s+2 are resident or on their way while slab s is multiplied.  A CU accepts one such copy
// instruction per 16 clocks, so a wave that issues its eight copies of a slab back to back stalls for hundreds
// of clocks and its matrix instructions with it: the copies are issued one at a time between matrix
// instructions.  Waits are counted: at the one barrier per slab a wave waits for its own copies of slab s + 1
// only (s_waitcnt vmcnt(4) leaves the four younger X_s+2 copies in flight).  Operand fragments are read one
// 16-column step ahead of the matrix instructions that use them.
//
// LDS rows are 128 bytes; the 16-byte piece c of row r is stored at slot c ^ ((r >> 1) & 7).  A ds_read_b128
// serves 16 lanes per clock from 64 banks (256 bytes); 16 consecutive rows of one piece then fall on 16
// different 16-byte bank groups ((r & 1) * 8 + slot), so the operand reads are conflict free.
//
// Operand layout of v_mfma_f32_32x32x16_f16, lane l: A row / B column l % 32, k = 8 * (l / 32) .. + 7;
// D[v], v = 0..15: row 8 * (v / 4) + 4 * (l / 32) + v % 4, column l % 32.  Rows of D are tokens, columns
// are weight rows, so a half-wave stores 32 consecutive outputs of one token.
#include "sq_common.h"

namespace sq {

constexpr int G_BM = 256, G_BN = 256, G_BK = 64, G_WAVES = 8;
constexpr int G_SLOTS = 5, G_SLOT_BYTES = 256 * G_BK * 2;        // 5 x 32 KB = all 160 KB of LDS

struct Gemm256Args {
    const uint16_t* x;        // fp16 [T, C], row stride ldx
    const uint16_t* w;        // fp16 [R, C], row stride ldw
    const uint16_t* row_scale;  // fp16 [R] or NULL (no scaling)
    void* y;
    int64_t ldx, ldw, ldy;
    int T, R, C, y_off, y_dtype;
    int tiles_t, tiles_r;     // token / weight-row tiles (for the workgroup -> tile mapping)
    // The last round of tiles rarely fills the chip (592 tiles on 256 CUs: 2 full rounds and 80 tiles).  Tiles
    // [0, main_tiles) are multiplied whole; each of the remaining tail tiles is split over kt workgroups, each
    // taking the slabs [kz nk / kt, (kz + 1) nk / kt) and leaving an unscaled fp32 partial tile in
    // part[(tail tile * kt + kz)][256][256] for gemm256_reduce_kernel.
    int main_tiles, kt;
    float* part;
    int vec_y;                // y rows allow 16-byte stores of 16-bit results (y 16-byte aligned, ldy % 8 == y_off % 8 == 0)
};

constexpr int G_EP_PITCH = 64 * 2 + 16;      // bytes per token row of a wave's 128 x 64 output tile in LDS

// s_waitcnt immediate that waits until at most n vector-memory operations are outstanding and leaves the
// other counters alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8)
constexpr int vmcnt_only(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

__global__ __launch_bounds__(G_WAVES * 64) void gemm256_kernel(Gemm256Args a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroups are dealt round-robin to the 8 XCDs (each with its own L2), so XCD x = blockIdx % 8 takes one
    // contiguous run of whole tiles (a weight tile is then fetched by one L2 only) and, after those, one
    // contiguous run of tail parts.  The grid is padded; surplus workgroups leave.
    const int ntiles = a.tiles_t * a.tiles_r;
    const int xcd = (int)(blockIdx.x & 7), jx = (int)(blockIdx.x >> 3);
    const int main_per = (a.main_tiles + 7) >> 3, parts = (ntiles - a.main_tiles) * a.kt, parts_per = (parts + 7) >> 3;
    int tile, kz = 0, nparts = 1;
    if (jx < main_per) {
        tile = xcd * main_per + jx;
        if (tile >= a.main_tiles) return;
    } else {
        const int pidx = xcd * parts_per + (jx - main_per);
        if (pidx >= parts) return;
        tile = a.main_tiles + pidx / a.kt;
        kz = pidx - (pidx / a.kt) * a.kt;
        nparts = a.kt;
    }
    // consecutive tiles walk the token tiles of one weight tile, so a weight tile is fetched from HBM once and
    // its re-reads hit L2 while the (small) activation matrix stays resident
    const int bt = tile % a.tiles_t, br = tile / a.tiles_t;
    const int t0 = bt * G_BM, r0 = br * G_BN;
    const int wm = (wave >> 2) * 128, wn = (wave & 3) * 64;

    float16v acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // Copies.  One global_load_lds_dwordx4 fills 1 KB = 8 LDS rows in lane order, so lane s lands in row
    // s >> 3, slot s & 7 of its block and therefore fetches the piece the swizzle puts there.  Wave w copies
    // rows 32 w .. 32 w + 31 of an operand slab: 4 instructions.  Global addresses are a uniform base (advanced
    // per slab) plus per-lane 32-bit element offsets computed once; rows past the matrix edge re-read the last
    // row (their outputs are never stored).  Half h = 2 s is X of slab s, h = 2 s + 1 is W of slab s; half h
    // lives in ring slot h % 5.
    const int lrow = lane >> 3, slot = lane & 7;
    uint32_t xo[4], wo[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int row = wave * 32 + j * 8 + lrow;
        const int c = slot ^ ((row >> 1) & 7);
        const int t = t0 + row < a.T ? row : a.T - 1 - t0;
        const int r = r0 + row < a.R ? row : a.R - 1 - r0;
        xo[j] = (uint32_t)(t * (int)a.ldx + c * 8);
        wo[j] = (uint32_t)(r * (int)a.ldw + c * 8);
    }
    const int nk_all = a.C / G_BK, k_begin = (int)((int64_t)kz * nk_all / nparts);
    const int nk = (int)((int64_t)(kz + 1) * nk_all / nparts) - k_begin;
    const uint16_t* xt = a.x + (int64_t)t0 * a.ldx + (int64_t)k_begin * G_BK;
    const uint16_t* wt = a.w + (int64_t)r0 * a.ldw + (int64_t)k_begin * G_BK;
    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    auto copy_x = [&](int s, int j) {
        __builtin_amdgcn_global_load_lds((gptr_t)(xt + s * G_BK + xo[j]),
                                         (lptr_t)(smem + ((2 * s) % G_SLOTS) * G_SLOT_BYTES + wave * 4096 + j * 1024), 16, 0, 0);
    };
    auto copy_w = [&](int s, int j) {
        __builtin_amdgcn_global_load_lds((gptr_t)(wt + s * G_BK + wo[j]),
                                         (lptr_t)(smem + ((2 * s + 1) % G_SLOTS) * G_SLOT_BYTES + wave * 4096 + j * 1024), 16, 0, 0);
    };

    // Fragments.  A lane reads row (lane & 31) + 32 i of its wave's rows, piece 2 kk + (lane >> 5); the swizzle
    // term depends on the row modulo 16 only and the column step kk only flips bits 5-6 of the offset, so one
    // offset per operand plus compile-time multiples of 32 rows (4096 bytes) covers all reads of a slab.
    half8v fa[2][4], fb[2][2];
    const int frow = lane & 31, fhalf = lane >> 5, fsw = (frow >> 1) & 7;
    const uint32_t fa_off = (uint32_t)((wm + frow) * 128 + ((fhalf ^ fsw) << 4));
    const uint32_t fb_off = (uint32_t)((wn + frow) * 128 + ((fhalf ^ fsw) << 4));
    auto load_frags = [&](int s, int kk, int set) {
        const unsigned char* pa = smem + ((2 * s) % G_SLOTS) * G_SLOT_BYTES + (fa_off ^ (uint32_t)(kk << 5));
        const unsigned char* pb = smem + ((2 * s + 1) % G_SLOTS) * G_SLOT_BYTES + (fb_off ^ (uint32_t)(kk << 5));
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[set][i] = *reinterpret_cast<const half8v*>(pa + i * 4096);
#pragma unroll
        for (int j = 0; j < 2; ++j) fb[set][j] = *reinterpret_cast<const half8v*>(pb + j * 4096);
    };
    auto mma_row = [&](int set, int i) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[set][i], fb[set][j], acc[i][j], 0, 0, 0);
    };
#ifndef SQ_SB
#define SQ_SB() __builtin_amdgcn_sched_barrier(0)
#endif

#pragma unroll
    for (int j = 0; j < 4; ++j) copy_x(0, j);
#pragma unroll
    for (int j = 0; j < 4; ++j) copy_w(0, j);
    if (nk > 1) {
#pragma unroll
        for (int j = 0; j < 4; ++j) copy_x(1, j);
        __builtin_amdgcn_s_waitcnt(vmcnt_only(4));
    } else {
        __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
    }
    __builtin_amdgcn_s_barrier();
    load_frags(0, 0, 0);
    for (int s = 0; s < nk; ++s) {
        // Each 16-column step starts with two matrix instructions (the wait in front of them covers only
        // fragment reads issued a whole step earlier), then requests the next step's fragments, then finishes
        // its matrix instructions with this slab's share of copies in between.
        const bool more1 = s + 1 < nk, more2 = s + 2 < nk;
        // step 0: W of slab s + 1 goes out first (it is needed at the end of this slab)
        mma_row(0, 0); SQ_SB();
        load_frags(s, 1, 1); SQ_SB();
        mma_row(0, 1); SQ_SB();
        if (more1) { copy_w(s + 1, 0); copy_w(s + 1, 1); } SQ_SB();
        mma_row(0, 2); SQ_SB();
        if (more1) copy_w(s + 1, 2); SQ_SB();
        mma_row(0, 3); SQ_SB();
        if (more1) copy_w(s + 1, 3); SQ_SB();
        // steps 1 and 2: X of slab s + 2
        mma_row(1, 0); SQ_SB();
        load_frags(s, 2, 0); SQ_SB();
        mma_row(1, 1); SQ_SB();
        if (more2) copy_x(s + 2, 0); SQ_SB();
        mma_row(1, 2); SQ_SB();
        if (more2) copy_x(s + 2, 1); SQ_SB();
        mma_row(1, 3); SQ_SB();
        mma_row(0, 0); SQ_SB();
        load_frags(s, 3, 1); SQ_SB();
        mma_row(0, 1); SQ_SB();
        if (more2) copy_x(s + 2, 2); SQ_SB();
        mma_row(0, 2); SQ_SB();
        if (more2) copy_x(s + 2, 3); SQ_SB();
        mma_row(0, 3); SQ_SB();
        // step 3: this wave's copies of slab s + 1 are waited for (the four X copies of slab s + 2 stay in
        // flight), then the barrier: everybody's copies of slab s + 1 have landed and everybody has read slab s
        // to the end, so its two slots can take W of slab s + 2 and X of slab s + 3 during the next slab
        mma_row(1, 0); SQ_SB();
        if (more1) {
            if (more2) __builtin_amdgcn_s_waitcnt(vmcnt_only(4)); else __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
            SQ_SB();
            __builtin_amdgcn_s_barrier();
            SQ_SB();
            load_frags(s + 1, 0, 0);
        }
        SQ_SB();
        mma_row(1, 1); mma_row(1, 2); mma_row(1, 3); SQ_SB();
    }
#undef SQ_SB

    // Epilogue.  In the accumulator layout a lane holds one weight row and 4 consecutive tokens, so direct stores
    // are 2-byte pieces (49 us of a 376 us product at the 2048 x 18944 output).  16-bit results therefore go
    // through the now idle LDS: every wave lays its 128 x 64 tile out token-major and writes it in 16-byte
    // pieces, 128 contiguous bytes per token.
    if (nparts == 1 && a.vec_y && a.y_dtype != SQ_F32) {
        __syncthreads();                                        // every wave is done with the operand ring
        unsigned char* my = smem + wave * (128 * G_EP_PITCH);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int rl = j * 32 + (lane & 31);
            const int r = r0 + wn + rl;
            const float sc_r = a.row_scale ? h2f(a.row_scale[r < a.R ? r : a.R - 1]) : 1.f;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int tl = i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                    const float val = acc[i][j][v] * sc_r;
                    *reinterpret_cast<uint16_t*>(my + tl * G_EP_PITCH + rl * 2) = a.y_dtype == SQ_BF16 ? f2bf(val) : f2h(val);
                }
        }
        uint16_t* yb = reinterpret_cast<uint16_t*>(a.y);
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const int idx = k * 64 + lane, tl = idx >> 3, piece = idx & 7;
            const int t = t0 + wm + tl, r = r0 + wn + piece * 8;
            if (t >= a.T || r >= a.R) continue;
            const u32x4 v = *reinterpret_cast<const u32x4*>(my + tl * G_EP_PITCH + piece * 16);
            uint16_t* dst = yb + (int64_t)t * a.ldy + a.y_off + r;
            if (r + 8 <= a.R) {
                *reinterpret_cast<u32x4*>(dst) = v;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (r + e < a.R) dst[e] = (uint16_t)(v[e >> 1] >> (16 * (e & 1)));
            }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int r = r0 + wn + j * 32 + (lane & 31);
        if (r >= a.R) continue;
        const float sc_r = a.row_scale ? h2f(a.row_scale[r]) : 1.f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int t = t0 + wm + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (t >= a.T) continue;
                if (nparts > 1) {
                    a.part[((int64_t)(tile - a.main_tiles) * a.kt + kz) * (G_BM * G_BN) + (t - t0) * G_BN + (r - r0)] = acc[i][j][v];
                    continue;
                }
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

// tail tiles: y[t, y_off + r] = row_scale[r] * sum over kz of part[(tail tile * kt + kz)][t - t0][r - r0]
__global__ __launch_bounds__(256) void gemm256_reduce_kernel(const float* __restrict__ part, int main_tiles, int kt, int tiles_t,
                                                             int T, int R, const uint16_t* __restrict__ row_scale, void* y,
                                                             int64_t ldy, int y_off, int y_dtype) {
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;      // element of a tail tile, 4 per thread
    const int tail = (int)(i / (G_BM * G_BN)), e = (int)(i - (int64_t)tail * (G_BM * G_BN));
    const int tile = main_tiles + tail, t = (tile % tiles_t) * G_BM + e / G_BN, r = (tile / tiles_t) * G_BN + e % G_BN;
    if (t >= T) return;
    const float* p = part + (int64_t)tail * kt * (G_BM * G_BN) + e;
    float4v sum = *reinterpret_cast<const float4v*>(p);
    for (int kz = 1; kz < kt; ++kz) sum += *reinterpret_cast<const float4v*>(p + (int64_t)kz * (G_BM * G_BN));
#pragma unroll
    for (int q = 0; q < 4; ++q)
        if (r + q < R) store_y(y, y_dtype, (int64_t)t * ldy + y_off + r + q, sum[q] * (row_scale ? h2f(row_scale[r + q]) : 1.f));
}

// How the tiles of a T x R output are dealt to `cus` CUs: whole rounds of whole tiles, and the tiles of the last,
// partial round split over kt workgroups each (kt = 1: no split) while a part keeps at least 16 slabs.
struct Gemm256Plan { int main_tiles, tail_tiles, kt; };
static Gemm256Plan gemm256_plan(int T, int R, int C, int cus) {
    const int tiles = ((T + G_BM - 1) / G_BM) * ((R + G_BN - 1) / G_BN);
    Gemm256Plan p{tiles, 0, 1};
    if (cus < 8) return p;
    const int main = tiles / cus * cus, tail = tiles - main;          // cus is a multiple of 8 on this hardware
    if (tail == 0 || main % 8) return p;
    // kt = the split with the least estimated time of the last round: rounds of workgroups x slabs per part, plus the
    // partial tiles written and read back (256 KB each way per part; a slab of a round takes about 1.45 us, a part's
    // reduction traffic about 0.12 us of the chip's memory bandwidth).  5120 x 17408 at 2048 rows (160 tiles): kt = 3
    // makes 480 workgroups, 1.9 rounds of a third of the slabs, 391 -> 318 us by this estimate.
    const int slabs = C / G_BK;
    int best = 1;
    double best_t = 1e30;
    for (int kt = 1; kt <= 4; ++kt) {
        if (kt > 1 && slabs / kt < 16) break;
        const int wgs = tail * kt, rounds = (wgs + cus - 1) / cus;
        const double t = rounds * (double)((slabs + kt - 1) / kt) * 1.45 + (kt > 1 ? wgs * 0.12 : 0.0);
        if (t < best_t - 1e-9) { best_t = t; best = kt; }
    }
    if (best < 2) return p;
    return Gemm256Plan{main, tail, best};
}

size_t gemm256_part_bytes(int T, int R, int C, int cus) {
    const Gemm256Plan p = gemm256_plan(T, R, C, cus);
    return ((size_t)p.tail_tiles * p.kt * G_BM * G_BN * 4 + 255) & ~(size_t)255;
}

bool gemm256_ok(int C, int64_t ldx, int64_t ldw, const void* x, const void* w) {
    return C % 64 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0;
}

// x and w fp16.  row_scale may be NULL.  `part` (gemm256_part_bytes) enables the split of the last round; NULL = no split.
int launch_gemm256(const uint16_t* x, int64_t ldx, const uint16_t* w, int64_t ldw, const uint16_t* row_scale, void* y,
                   int y_dtype, int64_t ldy, int y_off, int T, int R, int C, float* part, int cus, hipStream_t s) {
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
    const Gemm256Plan pl = part ? gemm256_plan(T, R, C, cus) : Gemm256Plan{a.tiles_t * a.tiles_r, 0, 1};
    a.main_tiles = pl.main_tiles;
    a.kt = pl.kt;
    a.part = part;
    a.vec_y = ((uintptr_t)y & 15) == 0 && ldy % 8 == 0 && y_off % 8 == 0;
    const unsigned grid = (unsigned)(8 * ((pl.main_tiles + 7) / 8 + (pl.tail_tiles * pl.kt + 7) / 8));
    hipLaunchKernelGGL(gemm256_kernel, dim3(grid), dim3(G_WAVES * 64), G_SLOTS * G_SLOT_BYTES, s, a);
    int rc = check_launch("sq_linear_gemm(gemm256)");
    if (rc || pl.tail_tiles == 0) return rc;
    const int64_t n4 = (int64_t)pl.tail_tiles * G_BM * G_BN / 4;
    hipLaunchKernelGGL(gemm256_reduce_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s, part, pl.main_tiles, pl.kt,
                       a.tiles_t, T, R, row_scale, y, ldy, y_off, y_dtype);
    return check_launch("sq_linear_gemm(gemm256 reduce)");
}

int launch_bf16_to_f16(const uint16_t* x, int64_t ldx, int T, int C, uint16_t* out, hipStream_t s) {
    const int64_t n = ((int64_t)T * C + 7) / 8;
    hipLaunchKernelGGL(bf16_to_f16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, x, ldx, T, C, out);
    return check_launch("sq_linear_gemm(bf16_to_f16)");
}

}  // namespace sq
