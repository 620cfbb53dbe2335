// Decode-time product of the d = 4 formats whose codebooks fit LDS (8-, 10- and 12-bit tags: 256, 1024 or 4096
// entries, up to four codebooks per matrix, no column orders) at 1 or 2 activation rows, straight from the file's
// row-major tags.
//
// A row is cut into segments of 16 x TPL tags; 16 lanes own a segment, lane j its tags TPL j .. TPL j + TPL - 1 (TPL = 8
// or 16 tags in whole dwords: 3 dwords for eight 12-bit tags, 5 for sixteen 10-bit tags, 4 or 2 for sixteen or eight
// 8-bit tags).  A workgroup's 16-lane groups are bound to (row slot, segment) pairs for the whole kernel: group g works
// on segment g mod nseg of row slot g / nseg, so the 4 TPL activations a lane multiplies with never change and stay in
// registers, and the four groups of a wave read consecutive bytes of a row per step.  Step t of a workgroup covers
// rows p0 + t rps .. + rps - 1 of its share [p0, p1) of the rows.  Per step a lane loads its dwords (six or eight
// steps are in flight per lane, requested before the codebook is staged), gathers TPL 8-byte codewords from the
// codebooks in LDS, adds 2 TPL two-element dot products, and the 16 lanes of a group add up with four DPP steps; the
// group's sum goes to its (row, segment) place in LDS.  No barrier inside the loop: after the last step one barrier,
// then the rows' segments are added in segment order, scaled and stored.  A row's sum is formed in the same order
// whatever the grid, the stack or the number of activation rows.
//
// Against the matrix-core kernel (sq_rows_mfma.h), whose registers hold one workgroup of 7 waves per CU and which needs
// a tile-major copy of the tags, this one reads the file's layout and holds every byte it will read of a small matrix
// in flight at once.
#include <atomic>
#include "sq_gemv_kernel.h"

namespace sq {

constexpr int SEG_MAX_PIECES = 4;
constexpr int SEG_MAX_WAVES = 16;
// Activation rows per launch.  Measured on the 7B-shaped layer (12-bit tags): two rows cost 55 us against 45 for one,
// four rows 85 (the matrix-core kernel: 58-60 at four).  The same products on the matrix cores
// (v_mfma_f32_4x4x4_16b_f16, one instruction per tag and activation row instead of two v_dot2c, element j of lane j's
// result) measured no faster at one or two rows (gate|up 17.0-17.5 / 21.0 against 16.8 / 20.6 us).
// Nor did a variant of this kernel for 3 to 8 rows that uses the whole instruction (the four lanes of a block take the same
// tags of four consecutive weight rows and one activation row each: four weight rows x four activation rows per
// instruction, a lane's registers hold one activation row's chunks as here): correct, and 53.3 / 55.3 / 60.8 us per
// 7B-shaped layer at 3 / 4 / 8 rows against 54.0 / 54.5 / 55.4 for the matrix-core kernel (gate|up 18.6 against 19.2, down
// 16.4-17.9 against 15.6).  With neither gathers, products nor sums (timing only) its gate|up launch still takes 16.9 us:
// what these launches wait for is the tags, which arrive at 4.2 TB/s.
constexpr int SEG_MAX_ROWS = 2;
constexpr int SEG_MAX_BOOKS = 4;                // codebooks per matrix (4 x 32 KB of the CU's 160 KB of LDS at 12 bits)

// Tags per lane and step, dwords that hold them, steps of tags in flight per lane (fewer where a step is wide or two
// activation rows are kept: registers)
template <int BITS, int TPL> struct seg_cfg {
    static constexpr int WPL = TPL * BITS / 32;
    static_assert(WPL * 32 == TPL * BITS, "a lane's tags fill whole dwords");
    static constexpr int pf(int NB) { return WPL >= 4 ? (NB > 1 ? 3 : WPL == 5 ? 5 : 6) : 8; }
    static constexpr uint32_t MASK = ((1u << BITS) - 1u) << 3;   // a tag times 8 bytes
};

struct SegPiece {
    const uint32_t* tags;
    const uint16_t* table;
    const uint16_t* row_scale;
    const uint8_t* row_book;             // codebook of every row (several codebooks per matrix) or NULL
    int R, y_off, wg_begin, wg_count;
};

struct SegArgs {
    SegPiece p[SEG_MAX_PIECES];
    int n;
    const uint16_t* x;                   // activation row b0
    void* y;                             // output row b0
    int64_t ldx, ldy;
    int nb;                              // activation rows of this launch (<= NB)
    int x_dtype, y_dtype;
    int W;                               // dwords per row of tags
    int nseg;                            // segments per row
    int rps;                             // rows per step of a workgroup
    int rows_max;                        // most rows in one workgroup's share: the LDS sums are [NB][rows_max][nseg]; the
                                         // activation rows follow them as fp16 [NB][C]
    int table_bytes;                     // all codebooks of a piece: G x 2^bits x 8 bytes
    int xdirect;                         // 1: no room in LDS for the activation rows, every lane fetches its own
};

typedef __attribute__((address_space(3))) void* seg_lptr_t;
typedef const __attribute__((address_space(1))) void* seg_gptr_t;
typedef __attribute__((address_space(3))) u32x2 seg_lds_u32x2;

// a lane's dwords of one step: the fewest loads that cover WPL dwords (4-byte aligned)
template <int WPL>
__device__ __forceinline__ dwords<WPL> seg_load(const uint32_t* p) {
    dwords<WPL> r;
    if constexpr (WPL == 2) {
        const u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
        r.v[0] = t.x; r.v[1] = t.y;
    } else if constexpr (WPL == 3) {
        const u32x3 t = __builtin_nontemporal_load(reinterpret_cast<const u32x3*>(p));
        r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z;
    } else if constexpr (WPL == 4) {
        const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
        r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
    } else {
        static_assert(WPL == 5, "2 to 5 dwords per lane and step");
        const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
        r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
        r.v[4] = __builtin_nontemporal_load(p + 4);
    }
    return r;
}

// LDS byte address of the codeword of tag k of a lane's dwords (the tag times 8, plus the offset of the row's
// codebook: `(v & mask) | offset` is one instruction); tag k sits at bit k BITS
template <int BITS, int WPL, int K>
__device__ __forceinline__ uint32_t seg_address(const dwords<WPL>& w, uint32_t bo) {
    constexpr int P = K * BITS, I = P >> 5, S = P & 31;
    constexpr uint32_t MASK = ((1u << BITS) - 1u) << 3;
    uint32_t v;
    if constexpr (S + BITS <= 32) v = S >= 3 ? w.v[I] >> (S - 3) : w.v[I] << (3 - S);
    else v = __builtin_amdgcn_alignbit(w.v[I + 1 < WPL ? I + 1 : I], w.v[I], S - 3);   // (a straddling tag starts past bit 3)
    return (v & MASK) | bo;
}

// NB activation rows; MB: rows name one of several codebooks (row_book), all of them in LDS
template <int BITS, int TPL, int NB, bool MB>
__global__ __launch_bounds__(SEG_MAX_WAVES * 64) void segs_kernel(SegArgs a) {
    typedef seg_cfg<BITS, TPL> F;
    constexpr int WPL = F::WPL, PF = F::pf(NB);
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = (int)blockDim.x >> 6;
    int pi = 0;
#pragma unroll
    for (int k = 1; k < SEG_MAX_PIECES; ++k)
        if (k < a.n && (int)blockIdx.x >= a.p[k].wg_begin) pi = k;
    const SegPiece P = a.p[pi];
    const int wg = (int)blockIdx.x - P.wg_begin;
    const int p0 = (int)((int64_t)P.R * wg / P.wg_count), p1 = (int)((int64_t)P.R * (wg + 1) / P.wg_count);
    const int nrows = p1 - p0;                                   // >= 1: the launcher makes no more workgroups than rows
    const int nseg = a.nseg, rps = a.rps;
    const int nsteps = (nrows + rps - 1) / rps;
    // (the codeword gathers form LDS addresses as numbers counted from the start of the dynamic LDS, which is address 0
    // in a kernel without static LDS; a build in which it is not leaves y unwritten, which no test survives)
    if ((uint32_t)(uintptr_t)(seg_lptr_t)lds != 0u) return;

    const int gidx = tid >> 4, j = tid & 15;
    const bool active = gidx < nseg * rps;                       // groups past the last (row slot, segment) pair shadow group 0
    const int g2 = active ? gidx : 0;
    const int rsub = g2 / nseg, seg = g2 - rsub * nseg;
    const uint32_t* tg = P.tags + (seg * 16 + j) * WPL;
    auto row_of = [&](int t) { return min(p0 + min(t, nsteps - 1) * rps + rsub, p1 - 1); };
    auto load_step = [&](int t) { return seg_load<WPL>(tg + (size_t)row_of(t) * a.W); };

    // Everything this workgroup needs from memory is requested before anything waits, in the order in which it can come
    // back (a wave's loads return in the order of their issue): the activation rows, which the cache holds, the
    // codebooks (memory to LDS without passing through registers; the last, partial KB through registers), the first
    // steps of tags, which come from memory.  (The activations requested behind the tags arrive behind them: 2.8 us of a
    // 46.8 us layer at one row.)
    // One activation row is fetched by every lane for itself (64 bytes, the 16 lanes of a group 1 KB in a row); two go
    // through LDS once per workgroup, 16 bytes per thread and turn, where every group of a segment finds them (fetched
    // per lane they would cost as much cache traffic as the tags).
    constexpr int XT = 4;                                        // turns requested together
    constexpr int XL = TPL / 2;                                  // 16-byte pieces of a row that one lane multiplies with
    const int xchunks = nseg * 16 * XL;                          // 16-byte pieces of a row
    unsigned char* xs = lds + a.table_bytes + (((size_t)NB * a.rows_max * nseg * 4 + 15) & ~(size_t)15);   // [NB][C] fp16
    u32x4 xown[NB][XL];                                          // (xdirect) this lane's activations as loaded
    if (a.xdirect) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const u32x4* xp = reinterpret_cast<const u32x4*>(a.x + (int64_t)min(b, a.nb - 1) * a.ldx) + (seg * 16 + j) * XL;
#pragma unroll
            for (int i = 0; i < XL; ++i) xown[b][i] = xp[i];
        }
    }
    const bool xearly = !a.xdirect && NB * xchunks <= XT * (int)blockDim.x;   // one turn serves the rows: its loads go out now
    u32x4 xv[XT];
    if (xearly) {
#pragma unroll
        for (int k = 0; k < XT; ++k) {
            const int i = min(tid + k * (int)blockDim.x, NB * xchunks - 1), b = i / xchunks;
            xv[k] = reinterpret_cast<const u32x4*>(a.x + (int64_t)min(b, a.nb - 1) * a.ldx)[i - b * xchunks];
        }
    }
    {
        const unsigned char* src = reinterpret_cast<const unsigned char*>(P.table);
        for (int c = wave; c < a.table_bytes / 1024; c += nwaves)
            __builtin_amdgcn_global_load_lds((seg_gptr_t)(src + (size_t)c * 1024 + lane * 16), (seg_lptr_t)(lds + c * 1024), 16, 0, 0);
    }
    dwords<WPL> ring[PF];
#pragma unroll
    for (int q = 0; q < PF; ++q) ring[q] = load_step(q);
    if (xearly) {
#pragma unroll
        for (int k = 0; k < XT; ++k) {
            const int i = tid + k * (int)blockDim.x;
            u32x4 q = xv[k];
            if (a.x_dtype == SQ_BF16) { q.x = bf2h_x2(q.x); q.y = bf2h_x2(q.y); q.z = bf2h_x2(q.z); q.w = bf2h_x2(q.w); }
            if (i < NB * xchunks) reinterpret_cast<u32x4*>(xs)[i] = q;
        }
    }
    for (int i0 = tid; !a.xdirect && !xearly && i0 < NB * xchunks; i0 += XT * (int)blockDim.x) {
        u32x4 v[XT];
#pragma unroll
        for (int k = 0; k < XT; ++k) {
            const int i = min(i0 + k * (int)blockDim.x, NB * xchunks - 1), b = i / xchunks;
            v[k] = reinterpret_cast<const u32x4*>(a.x + (int64_t)min(b, a.nb - 1) * a.ldx)[i - b * xchunks];
        }
#pragma unroll
        for (int k = 0; k < XT; ++k) {
            const int i = i0 + k * (int)blockDim.x;
            u32x4 q = v[k];
            if (a.x_dtype == SQ_BF16) { q.x = bf2h_x2(q.x); q.y = bf2h_x2(q.y); q.z = bf2h_x2(q.z); q.w = bf2h_x2(q.w); }
            if (i < NB * xchunks) reinterpret_cast<u32x4*>(xs)[i] = q;
        }
    }
    float* psum = reinterpret_cast<float*>(lds + a.table_bytes);   // [NB][rows_max][nseg]
    // several codebooks: the codebook ids of this workgroup's rows, one byte each, behind everything else in LDS
    unsigned char* lbooks = xs + (a.xdirect ? 0 : (size_t)NB * xchunks * 16);
    if (MB)
        for (int i = tid; i < nrows; i += (int)blockDim.x) lbooks[i] = P.row_book[p0 + i];
    if ((a.table_bytes & 1023) != 0) {                           // (codebooks of 256 entries: G x 2 KB is whole KB; kept for safety)
        const int done = a.table_bytes & ~1023;
        for (int i = done + tid * 4; i < a.table_bytes; i += (int)blockDim.x * 4)
            *reinterpret_cast<uint32_t*>(lds + i) = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const unsigned char*>(P.table) + i);
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    // LDS offset of the codebook of step t's row, read one step ahead of its use
    auto book_at = [&](int t) { return MB ? (uint32_t)lbooks[row_of(t) - p0] << (BITS + 3) : 0u; };
    uint32_t bo = book_at(0);
    uint32_t xr[NB][2 * TPL];                                    // this lane's 4 TPL activations per row, as fp16 pairs
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            u32x4 q;
            if (a.xdirect) {
                q = xown[b][i];
                if (a.x_dtype == SQ_BF16) { q.x = bf2h_x2(q.x); q.y = bf2h_x2(q.y); q.z = bf2h_x2(q.z); q.w = bf2h_x2(q.w); }
            } else {
                q = reinterpret_cast<const u32x4*>(xs + ((size_t)b * xchunks + (seg * 16 + j) * XL) * 16)[i];
            }
            xr[b][4 * i] = q.x; xr[b][4 * i + 1] = q.y; xr[b][4 * i + 2] = q.z; xr[b][4 * i + 3] = q.w;
        }

    // LDS byte addresses of the codewords of a lane's tags
    auto addresses = [](const dwords<WPL>& w, uint32_t bo_, uint32_t (&ad)[TPL]) {
        ad[0] = seg_address<BITS, WPL, 0>(w, bo_); ad[1] = seg_address<BITS, WPL, 1>(w, bo_);
        ad[2] = seg_address<BITS, WPL, 2>(w, bo_); ad[3] = seg_address<BITS, WPL, 3>(w, bo_);
        ad[4] = seg_address<BITS, WPL, 4>(w, bo_); ad[5] = seg_address<BITS, WPL, 5>(w, bo_);
        ad[6] = seg_address<BITS, WPL, 6>(w, bo_); ad[7] = seg_address<BITS, WPL, 7>(w, bo_);
        if constexpr (TPL == 16) {
            ad[8] = seg_address<BITS, WPL, 8>(w, bo_); ad[9] = seg_address<BITS, WPL, 9>(w, bo_);
            ad[10] = seg_address<BITS, WPL, 10>(w, bo_); ad[11] = seg_address<BITS, WPL, 11>(w, bo_);
            ad[12] = seg_address<BITS, WPL, 12>(w, bo_); ad[13] = seg_address<BITS, WPL, 13>(w, bo_);
            ad[14] = seg_address<BITS, WPL, 14>(w, bo_); ad[15] = seg_address<BITS, WPL, 15>(w, bo_);
        }
    };
    // the rest of a step: the codewords (eight gathers in flight at a time), their products, the group's sum to its place
    auto finish = [&](int t, const uint32_t (&ad)[TPL]) {
        float acc[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[b] = 0.f;
#pragma unroll
        for (int k0 = 0; k0 < TPL; k0 += 8) {
            u32x2 cw[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) cw[k] = *reinterpret_cast<const seg_lds_u32x2*>((uintptr_t)ad[k0 + k]);
#pragma unroll
            for (int k = 0; k < 8; ++k)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint32_t cwh = cw[k][h];               // (bit_cast straight from a vector element misreads it)
#pragma unroll
                    for (int b = 0; b < NB; ++b)
                        acc[b] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, cwh), __builtin_bit_cast(half2v, xr[b][2 * (k0 + k) + h]), acc[b], false);
                }
        }
        const int row = p0 + t * rps + rsub;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const float v = team_sum(acc[b], 16);                // every lane of the group holds the group's sum
            if (j == 15 && active && row < p1) psum[((size_t)b * a.rows_max + (row - p0)) * nseg + seg] = v;
        }
    };
    // Whole rounds of PF steps, then the rest.  Within a round a step's registers are refilled for the next round once
    // its addresses have been formed from them (the same registers: no copies at the end of a round, and no branch
    // inside one, so the waits count loads exactly).
    int t0 = 0;
    for (; t0 + PF <= nsteps; t0 += PF) {
#pragma unroll
        for (int q = 0; q < PF; ++q) {
            uint32_t ad[TPL];
            addresses(ring[q], bo, ad);
            __builtin_amdgcn_sched_barrier(0);
            ring[q] = load_step(t0 + q + PF);
            bo = book_at(t0 + q + 1);
            __builtin_amdgcn_sched_barrier(0);
            finish(t0 + q, ad);
        }
    }
#pragma unroll
    for (int q = 0; q < PF; ++q)
        if (t0 + q < nsteps) {                                   // uniform in the workgroup
            uint32_t ad[TPL];
            addresses(ring[q], bo, ad);
            bo = book_at(t0 + q + 1);
            finish(t0 + q, ad);
        }
    __syncthreads();
    const size_t ysz = a.y_dtype == SQ_F32 ? 4 : 2;
    for (int idx = tid; idx < nrows * a.nb; idx += (int)blockDim.x) {
        const int b = idx / nrows, rl = idx - b * nrows;
        const float* ps = psum + ((size_t)b * a.rows_max + rl) * nseg;
        float sum = 0.f;
        for (int sgi = 0; sgi < nseg; ++sgi) sum += ps[sgi];
        const int r = p0 + rl;
        store_y((char*)a.y + (size_t)b * a.ldy * ysz, a.y_dtype, (int64_t)P.y_off + r, sum * h2f(P.row_scale[r]));
    }
}

// Tags per lane and step for rows of U tags of `bits` bits: 16 x TPL tags per segment must divide the row (0: none does)
static int segs_tpl(int U, int bits) {
    if (bits == 12) return U % 128 == 0 ? 8 : 0;
    if (bits == 10) return U % 256 == 0 ? 16 : 0;
    if (bits == 8) return U % 256 == 0 ? 16 : U % 128 == 0 ? 8 : 0;
    return 0;
}

// d = 4, 8- / 10- / 12-bit tags, up to SEG_MAX_BOOKS codebooks (all of them fit LDS), no column orders, rows of whole
// segments, at most SEG_MAX_WAVES * 4 segments per row
bool segs_shape(const sq_matrix& m) {
    if (!m.tags || m.d != 4 || m.G < 1 || m.G > SEG_MAX_BOOKS || m.perms || m.R <= 0 || m.C % m.d) return false;
    if (m.G > 1 && !m.row_book) return false;
    const int U = m.C / m.d, tpl = segs_tpl(U, m.bits);
    if (!tpl || U / (16 * tpl) > SEG_MAX_WAVES * 4) return false;
    if ((int64_t)U * m.bits != (int64_t)m.W * 32) return false;
    return (((uintptr_t)m.tags & 15) | ((uintptr_t)m.table & 15)) == 0;   // (a lane's loads are dword-aligned, no more)
}

template <int BITS, int TPL, int NB, bool MB>
static int segs_launch_as(const SegArgs& a, int grid, int threads, size_t smem, hipStream_t s) {
    static std::atomic<bool> raised{false};
    if (!raised.load(std::memory_order_acquire)) {
        (void)hipFuncSetAttribute((const void*)segs_kernel<BITS, TPL, NB, MB>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        (void)hipGetLastError();
        raised.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL((segs_kernel<BITS, TPL, NB, MB>), dim3((unsigned)grid), dim3((unsigned)threads), smem, s, a);
    return check_launch("sq_linear_small(segs)");
}

template <int BITS, int TPL>
static int segs_launch_fmt(const SegArgs& a, int NB, bool mb, int grid, int threads, size_t smem, hipStream_t s) {
    if (mb) return NB == 1 ? segs_launch_as<BITS, TPL, 1, true>(a, grid, threads, smem, s) : segs_launch_as<BITS, TPL, 2, true>(a, grid, threads, smem, s);
    return NB == 1 ? segs_launch_as<BITS, TPL, 1, false>(a, grid, threads, smem, s) : segs_launch_as<BITS, TPL, 2, false>(a, grid, threads, smem, s);
}

// How pieces [0, cnt) (same C, same tag width, same number of codebooks) are launched together: false when the
// workgroups' partial sums would not fit LDS beside the codebooks (matrices of several hundred thousand rows).
struct SegPlan {
    int tpl, nseg, rps, waves, per_cu, grid, rows_max, NB, table_bytes, xdirect;
    int wg_begin[SEG_MAX_PIECES], wg_count[SEG_MAX_PIECES];
    size_t smem;
};

static bool segs_plan(const sq_matrix* mats, int cnt, int B, int cus, SegPlan& pl) {
    const int U = mats[0].C / mats[0].d;
    pl.tpl = segs_tpl(U, mats[0].bits);
    if (!pl.tpl) return false;
    pl.nseg = U / (16 * pl.tpl);
    pl.table_bytes = mats[0].G * (8 << mats[0].bits);
    // 16-lane groups per workgroup: about 32 in 8 waves, two workgroups per CU, when the codebooks leave room for two;
    // about 64 in one workgroup of 16 waves otherwise
    const bool two = pl.table_bytes <= 64 * 1024;
    pl.rps = 8;
    while (pl.rps > 1 && pl.nseg * pl.rps > (two ? 32 : 64)) pl.rps >>= 1;
    pl.waves = (pl.nseg * pl.rps + 3) / 4;
    pl.NB = B;
    int64_t rows_total = 0;
    for (int k = 0; k < cnt; ++k) rows_total += mats[k].R;
    for (pl.per_cu = two && pl.waves <= 8 ? 2 : 1; pl.per_cu >= 1; --pl.per_cu) {   // workgroups a CU holds (128 registers per lane)
        pl.grid = 0;
        pl.rows_max = 1;
        for (int k = 0; k < cnt; ++k) {
            const int R = mats[k].R;
            int64_t n = (int64_t)R * cus * pl.per_cu / rows_total;   // (rounded down: one workgroup too many is a second round)
            const int64_t most = (R + pl.rps - 1) / pl.rps;      // a workgroup has at least one full step
            if (n > most) n = most;
            if (n < 1) n = 1;
            pl.wg_begin[k] = pl.grid;
            pl.wg_count[k] = (int)n;
            pl.grid += (int)n;
            pl.rows_max = std::max(pl.rows_max, (int)((R + n - 1) / n));
        }
        const size_t room = (size_t)(160 * 1024) / pl.per_cu;
        const size_t base = (size_t)pl.table_bytes + (((size_t)pl.NB * pl.rows_max * pl.nseg * 4 + 15) & ~(size_t)15);
        const size_t xs = (size_t)pl.NB * mats[0].C * 2;         // the activation rows as fp16
        const size_t ids = mats[0].G > 1 ? (((size_t)pl.rows_max + 15) & ~(size_t)15) : 0;   // codebook ids of the rows
        pl.xdirect = base + xs + ids > room || B == 1 ? 1 : 0;  // (one row: fetched per lane, 41.8 against 43.2 us per 7B-shaped layer)  // (one row: 45.0 against 46.8 us per 7B-shaped layer fetched per lane)
        pl.smem = base + (pl.xdirect ? 0 : xs) + ids;
        if (pl.smem <= room) return true;
    }
    return false;
}

bool segs_fits(const sq_matrix* mats, int cnt, int B, int cus) {
    SegPlan pl;
    return cnt >= 1 && cnt <= SEG_MAX_PIECES && B >= 1 && B <= SEG_MAX_ROWS && segs_plan(mats, cnt, B, cus, pl);
}

// Pieces [0, cnt) pass segs_shape, share C, the tag width and G, and segs_fits() holds (B <= SEG_MAX_ROWS); x is
// 16-byte aligned with ldx % 8 == 0.
int launch_segs_group(const sq_matrix* mats, int cnt, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                      int64_t ldy, int B, int cus, hipStream_t s) {
    SegPlan pl;
    if (!segs_fits(mats, cnt, B, cus) || !segs_plan(mats, cnt, B, cus, pl)) return fail(SQ_ELAUNCH, "sq_linear_small(segs): no plan");
    SegArgs a;
    a.n = cnt;
    a.x = (const uint16_t*)x; a.y = y; a.ldx = ldx; a.ldy = ldy; a.nb = B; a.x_dtype = x_dtype; a.y_dtype = y_dtype;
    a.W = mats[0].W;
    a.nseg = pl.nseg;
    a.rps = pl.rps;
    a.rows_max = pl.rows_max;
    a.table_bytes = pl.table_bytes;
    a.xdirect = pl.xdirect;
    for (int k = 0; k < cnt; ++k) {
        const sq_matrix& m = mats[k];
        SegPiece& P = a.p[k];
        P.tags = (const uint32_t*)m.tags; P.table = m.table; P.row_scale = m.row_scale; P.row_book = m.G > 1 ? m.row_book : nullptr;
        P.R = m.R; P.y_off = m.y_off;
        P.wg_begin = pl.wg_begin[k];
        P.wg_count = pl.wg_count[k];
    }
    for (int k = cnt; k < SEG_MAX_PIECES; ++k) a.p[k] = a.p[0];
    const int threads = pl.waves * 64, bits = mats[0].bits;
    const bool mb = mats[0].G > 1;
    if (bits == 12) return segs_launch_fmt<12, 8>(a, pl.NB, mb, pl.grid, threads, pl.smem, s);
    if (bits == 10) return segs_launch_fmt<10, 16>(a, pl.NB, mb, pl.grid, threads, pl.smem, s);
    if (pl.tpl == 16) return segs_launch_fmt<8, 16>(a, pl.NB, mb, pl.grid, threads, pl.smem, s);
    return segs_launch_fmt<8, 8>(a, pl.NB, mb, pl.grid, threads, pl.smem, s);
}

}  // namespace sq
