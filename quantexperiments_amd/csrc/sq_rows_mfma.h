// Decode-time codebook product on the matrix cores, B = 1..32 activation rows, for gfx950.
//
// v_mfma_f32_16x16x32_f16 multiplies a 16 x 32 tile of weights (A) by 32 x 16 activations (B):
//   A: lane l supplies row l % 16, 8 consecutive k starting at 8 * (l / 16)
//   B: lane l supplies activation row (token) l % 16, the same 8 k
//   D: lane l holds token l % 16, weight rows 4 * (l / 16) .. + 3
// Eight consecutive k of one weight row are exactly two d = 4 codewords or one d = 8 codeword, so a
// lane builds its A operand by gathering raw fp16 codewords (from LDS when the codebook fits) with no
// arithmetic at all, the sum over k happens inside the accumulator, and the cost of a tile does not
// depend on how many of the 16 activation rows are real.  The row scale multiplies the fp32 result.
//
// Work split.  A wave owns a slice of the columns for its whole life, so its B operands (the
// activations of that slice, converted bf16 -> fp16 once) are loaded once and stay in registers; it
// walks over 16-row tiles with the tags of the next tiles in flight (one tile ahead when the codewords come
// through the cache, which is then the bound; two or three tiles when the codebook sits in LDS).
// The tag stream is read in lane units (UD dwords = TPU whole tags = UK columns): in round n the four
// lane groups g = 0..3 of a row read units 4n + g, one wide load each, and the round's SPU matrix
// instructions consume the units chunk pair by chunk pair.  The KW waves of a workgroup split the
// columns of a tile; their accumulators are added through LDS by one wave per tile (round robin): after
// every MMA_TT tiles when the codebook is read through the cache, after all the tiles of the workgroup (as
// many as LDS holds accumulators for: MmaArgs.tg) when it sits in LDS, so that the waves of a launch of the
// 7B shapes meet once.  Rows longer than KW * RW rounds are split over `ks` workgroups whose
// partial sums go to a workspace and are added, in slice order, by splitk_reduce_kernel.
#pragma once
#include <mutex>
#include <unordered_map>
#include "sq_gemv_kernel.h"

namespace sq {

struct MmaPiece {
    sq_matrix m;
    const uint32_t* tiled; // tile-major copy of the tags (sq_matrix.stream of a d = 4 format) or NULL
    float* part;          // ks > 1: fp32 [ks, B, R] unscaled partial sums of this piece
    int wg_begin;         // first workgroup of this piece
    int wg_count;         // nshare * ks workgroups
};

struct MmaArgs {
    MmaPiece p[GEMV_MAX_PIECES];
    int n;
    const uint16_t* x;
    int64_t ldx;
    void* y;
    int64_t ldy;
    int B;
    int x_dtype, y_dtype;
    int U;                // lane units per row
    int ks;               // workgroup-level column slices
    int table_bytes;      // bytes of codebook staged in LDS (0 = read through cache)
    int tg;               // codebook in LDS: 16-row tiles whose accumulators LDS holds between two barriers (a multiple of mma_pft(RW))
};

constexpr int MMA_TT = 4;     // 16-row tiles multiplied between two workgroup barriers (codebook read through the cache)
// codebook in LDS: tiles of tags in flight per lane (fewer when a lane's part of a tile is long: registers)
// (2 to 5 tiles in flight measure alike on the 7B shapes)
constexpr int mma_pft(int RW) { return RW >= 8 ? 2 : 3; }
// LDS per wave in which a round's activations (16 tokens x 4 lane units of UK columns, fp16) pass from whole-line loads
// to the lanes that use them; it lies where the accumulators are added afterwards
constexpr int mma_x_stage_bytes(int UK) { return 16 * (4 * UK * 2 + 16); }

// Optional timeline of the first wave of every workgroup (debug builds define SQ_TRACE_POINT).
#ifndef SQ_TRACE_POINT
#define SQ_TRACE_POINT(k)
#endif

// LDS byte offset of the codeword of tag t of a unit, counted from the start of the dynamic LDS: the tag times 2^SH (the
// codeword size) plus `bo`, the byte offset of the row's codebook, whose bits lie above the tag's: one shift (or
// v_alignbit_b32 for a tag that straddles two dwords, which starts past bit SH) and one v_and_or_b32
template <int BITS, int UD, int SH>
__device__ __forceinline__ uint32_t unit_lds_offset(const dwords<UD>& u, int t, uint32_t bo) {
    const int p = t * BITS, w = p >> 5, s = p & 31;
    constexpr uint32_t MASK = ((1u << BITS) - 1u) << SH;
    uint32_t v;
    if (s + BITS <= 32) v = s >= SH ? u.v[w] >> (s - SH) : u.v[w] << (SH - s);
    else v = __builtin_amdgcn_alignbit(u.v[w + 1 < UD ? w + 1 : w], u.v[w], s - SH);
    return (v & MASK) | bo;
}
typedef __attribute__((address_space(3))) u32x2 mma_lds_u32x2;
typedef __attribute__((address_space(3))) u32x4 mma_lds_u32x4;

// two packed bf16 -> two packed fp16: round to nearest even like every other kernel of the library (exact for every
// fp16-normal value, +-inf beyond 65,504; a round-toward-zero conversion would clamp to 65,504 instead and make this
// kernel differ from the batch-1 one on the same input)
__device__ __forceinline__ uint32_t bf2h_pk(uint32_t v) { return bf2h_x2(v); }

// Waves per workgroup: up to 16 for the variants whose lanes hold at most 8 activation operands (32 registers) beside a
// codebook in LDS, which fit four waves per SIMD; 8 otherwise.
constexpr int mma_waves_max(int x_operands, bool lds_tab) { return lds_tab && x_operands <= 8 ? 16 : 8; }

template <int BITS, int D, int RW, int NT, bool LDS_TAB>
__global__ __launch_bounds__(64 * mma_waves_max(RW * ((unit_of<BITS>::UD * 32 / BITS) / (8 / D)) * NT, LDS_TAB))
void rows_mfma_kernel(MmaArgs a) {
    constexpr int UD = unit_of<BITS>::UD;
    constexpr int TPU = UD * 32 / BITS;      // tags per lane unit
    constexpr int CPS = 8 / D;               // codewords a lane feeds into one matrix instruction
    constexpr int SPU = TPU / CPS;           // matrix instructions per round
    constexpr int UK = TPU * D;              // columns per lane unit
    constexpr int ESZ = D * 2;               // bytes per codeword
    constexpr int TT = MMA_TT;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, li = lane & 15, lg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), KW = blockDim.x >> 6;
    int pi = 0;
    while (pi + 1 < a.n && (int)blockIdx.x >= a.p[pi + 1].wg_begin) ++pi;
    const MmaPiece& P = a.p[pi];
    const sq_matrix& m = P.m;
    const int w = blockIdx.x - P.wg_begin, slice = w % a.ks, share = w / a.ks, nshare = P.wg_count / a.ks;
    const int ntiles = (m.R + 15) >> 4;
    const int t0 = (int)((int64_t)ntiles * share / nshare), t1 = (int)((int64_t)ntiles * (share + 1) / nshare);
    SQ_TRACE_POINT(0);

    // LDS: [codebook][16 bytes, unused][reduction buffer: TT tiles x KW waves x 64 lanes x NT x 16 bytes]
    // (the codeword gathers form LDS addresses as numbers counted from the start of the dynamic LDS, which is address 0 in a
    // kernel without static LDS; a build in which it is not leaves y unwritten, which no test survives)
    if (LDS_TAB && (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)smem != 0u) return;
    float4v* red = reinterpret_cast<float4v*>(smem + a.table_bytes + 16);

    // ---- this wave's rounds
    const int rbase = (slice * KW + wave) * RW;
    bool live[RW];
    bool lane_live = true;
    uint32_t uoff[RW];
    int ucol[RW];
#pragma unroll
    for (int n = 0; n < RW; ++n) {
        const int u = 4 * (rbase + n) + lg;
        live[n] = u < a.U;
        lane_live = lane_live && live[n];
        const int uc = live[n] ? u : a.U - 1;
        uoff[n] = (uint32_t)uc * UD;
        ucol[n] = uc * UK;
    }
    // Units past the row's end (only in waves that cover the tail of the columns) contribute exact zeros: their
    // activation operands are zero, and what they multiply with is the row's own last unit again (with the codebook in
    // LDS; a codeword that is not finite is already part of the row's sum) or a zeroed operand (without).
    const bool all_live = __builtin_amdgcn_readfirstlane(__all(lane_live) ? 1 : 0) != 0;
    const uint32_t* tags = reinterpret_cast<const uint32_t*>(m.tags);
    const unsigned char* table = reinterpret_cast<const unsigned char*>(m.table);

    // ---- a tile's memory: tags of this lane's row, its codebook offset, the scales of its four output rows
    // (book: the byte of row_book as loaded; without codebook ids a byte of valid memory that `bkmask` turns into 0 where it is
    // used: a branch around the load, or a use right behind it, would make every wait of the loop a wait for all loads)
    struct Tile { dwords<UD> t[RW]; uint32_t book; };
    const uint8_t* bkp = m.row_book ? m.row_book : reinterpret_cast<const uint8_t*>(m.row_scale);
    const uint32_t bkmask = m.row_book ? 0xFFu : 0u;
    auto fetch = [&](int t, Tile& T, float (&sc)[4]) {
        const int row0 = t << 4;
        const int r = row0 + li < m.R ? row0 + li : m.R - 1;
        T.book = bkp[r];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int ro = row0 + 4 * lg + v;
            sc[v] = h2f(m.row_scale[ro < m.R ? ro : m.R - 1]);
        }
        if (P.tiled) {           // unit u of the tile's 16 rows: 16 * UD consecutive dwords
            const uint32_t* tp = P.tiled + ((size_t)t * a.U * 16 + li) * UD;
#pragma unroll
            for (int n = 0; n < RW; ++n) T.t[n] = load_unit<UD>(tp + (size_t)uoff[n] * 16);
        } else {
            const uint32_t* rp = tags + (size_t)r * m.W;
#pragma unroll
            for (int n = 0; n < RW; ++n) T.t[n] = load_unit<UD>(rp + uoff[n]);
        }
        if (!LDS_TAB && !all_live) {
#pragma unroll
            for (int n = 0; n < RW; ++n)
#pragma unroll
                for (int i = 0; i < UD; ++i) T.t[n].v[i] = live[n] ? T.t[n].v[i] : 0u;
        }
    };

    // ---- start-up: every load the first products need is requested before anything waits, in the order in which it
    // can come back (a wave's loads return in the order of their issue): the activations of this wave's columns, which
    // the cache holds; the tags of the first tiles, which come from memory; then, once the activations have been handed
    // to the lanes (a wait for them alone), the codebook.
    Tile tA, tB;
    float sc[TT + 1][4];                                      // [TT]: first tile of the next group, fetched early
    const bool table_dma = LDS_TAB && (a.table_bytes & 1023) == 0;
    // The activations.  In the matrix instruction a lane supplies one token's 8 columns, so loading the operands where
    // they are used makes every load instruction touch 64 different cache lines (16 tokens x 4 lane units, 16 bytes of
    // each).  Instead the wave fetches the columns of a round, 16 tokens x XRB contiguous bytes, with whole-line loads
    // (1 KB per instruction: 8 lines), and the lanes pick their operands out of LDS: a staging area per wave that lies
    // where the accumulators are added later, which nobody writes before the barrier below.
    constexpr int XRB = 4 * UK * 2;                          // bytes of one token's columns in one round of a wave
    constexpr int XROW = XRB + 16;                           // a token's row in the staging area (the 16 tokens' reads spread over the banks)
    constexpr int XTPI = 1024 / XRB;                         // tokens per load instruction
    static_assert(16 / XTPI == SPU, "a round's activations are SPU loads per token tile");
    unsigned char* xst = smem + a.table_bytes + 16 + wave * mma_x_stage_bytes(UK);
    const int xtl = lane / (XRB / 16), xob = (lane % (XRB / 16)) * 16;    // this lane's token (within an instruction) and byte in the round
    u32x4 xraw[RW][NT][SPU];
#pragma unroll
    for (int n = 0; n < RW; ++n)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int j = 0; j < SPU; ++j) {
                const int tok = nt * 16 + j * XTPI + xtl;
                int col = 4 * (rbase + n) * UK + (xob >> 1);
                col = col < m.C ? col : m.C - 8;             // (columns past the row's end: any valid address, the operand is zeroed)
                xraw[n][nt][j] = *reinterpret_cast<const u32x4*>(a.x + (int64_t)(tok < a.B ? tok : a.B - 1) * a.ldx + col);
            }
    fetch(t0 < t1 ? t0 : ntiles - 1, tA, sc[0]);             // (no branch around the loads; a workgroup without tiles reads the last one)
    // (codebook in LDS: the tags of the first tiles in flight, without a branch around the loads so that the waits count
    // them exactly: the two layouts differ in a base and a stride, chosen once)
    constexpr int PFT = LDS_TAB ? mma_pft(RW) : 1;
    const bool til = P.tiled != nullptr;
    const uint32_t* fbase = til ? P.tiled + li * UD : tags;
    uint32_t fo[RW];
#pragma unroll
    for (int n = 0; n < RW; ++n) fo[n] = til ? uoff[n] * 16u : uoff[n];
    auto fetch_tags = [&](int t, Tile& T) {
        const int row0 = t << 4;
        const int r = row0 + li < m.R ? row0 + li : m.R - 1;
        const uint32_t* bp = fbase + (til ? (size_t)t * a.U * 16 * UD : (size_t)r * m.W);
        T.book = bkp[r];                                  // (first: loads return in order, the tags' waits then cover it)
#pragma unroll
        for (int n = 0; n < RW; ++n) T.t[n] = load_unit<UD>(bp + fo[n]);
    };
    Tile ring[PFT];
    if constexpr (LDS_TAB) {
        ring[0] = tA;
#pragma unroll
        for (int q = 1; q < PFT; ++q) fetch_tags(min(t0 + q, max(t1 - 1, t0)), ring[q]);
    }
    // the B operands: this wave's activations as fp16, in registers for the whole kernel
    half8v xb[RW][SPU][NT];
#pragma unroll
    for (int n = 0; n < RW; ++n)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
            for (int j = 0; j < SPU; ++j) {
                u32x4 v = xraw[n][nt][j];
                if (a.x_dtype == SQ_BF16) { v.x = bf2h_pk(v.x); v.y = bf2h_pk(v.y); v.z = bf2h_pk(v.z); v.w = bf2h_pk(v.w); }
                *reinterpret_cast<u32x4*>(xst + (j * XTPI + xtl) * XROW + xob) = v;
            }
            // (the lanes of a wave exchange data here: its LDS instructions run in order, the fences keep the compiler from
            // moving a lane's reads before its writes)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int s = 0; s < SPU; ++s) {
                u32x4 v = *reinterpret_cast<const u32x4*>(xst + li * XROW + lg * (UK * 2) + s * 16);
                if (!(live[n] && nt * 16 + li < a.B)) v = u32x4{0u, 0u, 0u, 0u};
                xb[n][s][nt] = __builtin_bit_cast(half8v, v);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    // (a codebook of whole KB goes memory -> LDS without passing through registers, a wave instruction per KB)
    if (table_dma) {
        typedef const __attribute__((address_space(1))) void* gptr_t;
        typedef __attribute__((address_space(3))) void* lptr_t;
        for (int c = wave; c < (a.table_bytes >> 10); c += KW)
            __builtin_amdgcn_global_load_lds((gptr_t)(table + (size_t)c * 1024 + lane * 16), (lptr_t)(smem + c * 1024), 16, 0, 0);
    } else if (LDS_TAB) {
        stage_table(m.table, a.table_bytes, smem);
    }
    SQ_TRACE_POINT(1);
    // every wave has taken its operands out of the staging area (and, with the codebook in LDS, the codebook has landed
    // and the first tile's tags with it)
    __builtin_amdgcn_s_waitcnt(0);
    if (LDS_TAB || KW > 1) __syncthreads();
    SQ_TRACE_POINT(2);

    // One tile: NS = RW * SPU matrix instructions.  The codeword gathers run PD instructions ahead of the
    // matrix instruction that consumes them, so LDS latency overlaps the multiplies of earlier steps.
    constexpr int NS = RW * SPU, PD = NS < 6 ? NS : 6;
    auto multiply = [&](const Tile& cur, float4v (&acc)[NT]) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[nt] = float4v{0.f, 0.f, 0.f, 0.f};
        u32x4 av[NS];
        auto gather = [&](int k) {
            const int n = k / SPU, s = k - n * SPU;
            const bool dead = !all_live && !live[n];
            const uint32_t bo = ((cur.book & bkmask) << BITS) * ESZ;    // byte offset of the row's codebook
            if (D == 8) {
                if (LDS_TAB) {
                    av[k] = *reinterpret_cast<const mma_lds_u32x4*>((uintptr_t)unit_lds_offset<BITS, UD, 4>(cur.t[n], s, bo));
                } else {
                    const uint32_t tag = unit_tag<BITS, UD>(cur.t[n], s);
                    av[k] = *reinterpret_cast<const u32x4*>(table + ((size_t)tag * ESZ + bo));
                }
            } else {
                u32x2 c0, c1;
                if (LDS_TAB) {
                    c0 = *reinterpret_cast<const mma_lds_u32x2*>((uintptr_t)unit_lds_offset<BITS, UD, 3>(cur.t[n], 2 * s, bo));
                    c1 = *reinterpret_cast<const mma_lds_u32x2*>((uintptr_t)unit_lds_offset<BITS, UD, 3>(cur.t[n], 2 * s + 1, bo));
                } else {
                    const uint32_t g0 = unit_tag<BITS, UD>(cur.t[n], 2 * s);
                    const uint32_t g1 = unit_tag<BITS, UD>(cur.t[n], 2 * s + 1);
                    c0 = *reinterpret_cast<const u32x2*>(table + ((size_t)g0 * ESZ + bo));
                    c1 = *reinterpret_cast<const u32x2*>(table + ((size_t)g1 * ESZ + bo));
                }
                av[k] = u32x4{c0.x, c0.y, c1.x, c1.y};
            }
            if (!LDS_TAB && dead) av[k] = u32x4{0u, 0u, 0u, 0u};
        };
#pragma unroll
        for (int k = 0; k < PD; ++k) gather(k);
#pragma unroll
        for (int k = 0; k < NS; ++k) {
            if (k + PD < NS) gather(k + PD);
            __builtin_amdgcn_sched_barrier(0);          // keep the gathers ahead of the multiply they are not for
            const int n = k / SPU, s = k - n * SPU;
            const half8v af = __builtin_bit_cast(half8v, av[k]);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
                acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, xb[n][s][nt], acc[nt], 0, 0, 0);
        }
    };

    if constexpr (LDS_TAB) {
        // ---- codebook in LDS.  Nothing here waits for the cache, so what bounds the kernel is how many bytes of tags it
        // keeps in flight and how often its waves meet: every lane holds mma_pft(RW) tiles of tags (a tile's registers are
        // refilled as soon as its last codeword has been gathered), a tile's accumulator goes straight to its place in
        // LDS, and the waves meet once per a.tg tiles (once per launch when the workgroup's tiles all fit), after which
        // each tile is added up by one wave (round robin), scaled and stored.
        if (t0 >= t1) return;                                 // (uniform in the workgroup; the launcher gives every one a tile)
        auto tile_done = [&](int tl, const float4v (&acc)[NT]) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) red[((tl * KW + wave) * 64 + lane) * NT + nt] = acc[nt];
        };
        for (int tg = t0; tg < t1; tg += a.tg) {
            const int te = min(tg + a.tg, t1);
            if (tg > t0) __syncthreads();                     // the previous group's sums have been read
            int t = tg;
            for (; t + PFT <= te; t += PFT) {
#pragma unroll
                for (int q = 0; q < PFT; ++q) {
                    float4v acc[NT];
                    multiply(ring[q], acc);
                    __builtin_amdgcn_sched_barrier(0);
                    fetch_tags(min(t + q + PFT, t1 - 1), ring[q]);
                    __builtin_amdgcn_sched_barrier(0);
                    tile_done(t + q - tg, acc);
                }
            }
#pragma unroll
            for (int q = 0; q < PFT; ++q)
                if (t + q < te) {                             // (the last group's last tiles: nothing left to fetch)
                    float4v acc[NT];
                    multiply(ring[q], acc);
                    tile_done(t + q - tg, acc);
                }
            __syncthreads();
            for (int tl = wave; tl < te - tg; tl += KW) {
                const int row0 = (tg + tl) << 4;
                float scl[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int ro = row0 + 4 * lg + v;
                    scl[v] = h2f(m.row_scale[ro < m.R ? ro : m.R - 1]);
                }
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    float4v s4 = red[((tl * KW) * 64 + lane) * NT + nt];
                    for (int k = 1; k < KW; ++k) {
                        const float4v o = red[((tl * KW + k) * 64 + lane) * NT + nt];
                        s4.x += o.x; s4.y += o.y; s4.z += o.z; s4.w += o.w;
                    }
                    const int tok = nt * 16 + li;
                    if (tok >= a.B) continue;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int r = row0 + 4 * lg + v;
                        if (r >= m.R) continue;
                        if (a.ks > 1) P.part[((int64_t)slice * a.B + tok) * m.R + r] = s4[v];
                        else store_y(a.y, a.y_dtype, (int64_t)tok * a.ldy + m.y_off + r, s4[v] * scl[v]);
                    }
                }
            }
        }
    } else {
        // ---- groups of TT tiles: multiply them one after the other (the next tile's tags load meanwhile), then
        // add the KW waves' accumulators through LDS, each tile of the group by a different wave
        for (int tg = t0, grp = 0; tg < t1; tg += TT, ++grp) {
            float4v acc[TT][NT];
            if (grp > 0) {
    #pragma unroll
                for (int v = 0; v < 4; ++v) sc[0][v] = sc[TT][v];
            }
    #pragma unroll
            for (int tt = 0; tt < TT; tt += 2) {
                if (tg + tt < t1) {
                    if (tg + tt + 1 < t1) fetch(tg + tt + 1, tB, sc[tt + 1]);
                    multiply(tA, acc[tt]);
                }
                if (tg + tt + 1 < t1) {
                    if (tg + tt + 2 < t1) fetch(tg + tt + 2, tA, sc[tt + 2]);
                    multiply(tB, acc[tt + 1]);
                }
            }
            SQ_TRACE_POINT(3 + 3 * (grp < 4 ? grp : 4));
            if (KW > 1) {
                if (grp > 0) __syncthreads();                     // the previous group's reducers are done reading
    #pragma unroll
                for (int tt = 0; tt < TT; ++tt)
    #pragma unroll
                    for (int nt = 0; nt < NT; ++nt) red[((tt * KW + wave) * 64 + lane) * NT + nt] = acc[tt][nt];
                __syncthreads();
            }
            SQ_TRACE_POINT(4 + 3 * (grp < 4 ? grp : 4));
    #pragma unroll
            for (int tt = 0; tt < TT; ++tt) {
                const int t = tg + tt;
                if (t >= t1) continue;
                if (KW > 1 && wave != (tt + grp) % KW) continue;   // this tile's reducer
                float4v tot[NT];
    #pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    if (KW > 1) {
                        float4v s4 = red[((tt * KW) * 64 + lane) * NT + nt];
                        for (int k = 1; k < KW; ++k) {
                            const float4v o = red[((tt * KW + k) * 64 + lane) * NT + nt];
                            s4.x += o.x; s4.y += o.y; s4.z += o.z; s4.w += o.w;
                        }
                        tot[nt] = s4;
                    } else tot[nt] = acc[tt][nt];
                }
                const int row0 = t << 4;
    #pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const int tok = nt * 16 + li;
                    if (tok >= a.B) continue;
    #pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int r = row0 + 4 * lg + v;
                        if (r >= m.R) continue;
                        if (a.ks > 1) P.part[((int64_t)slice * a.B + tok) * m.R + r] = tot[nt][v];
                        else store_y(a.y, a.y_dtype, (int64_t)tok * a.ldy + m.y_off + r, tot[nt][v] * sc[tt][v]);
                    }
                }
            }
            SQ_TRACE_POINT(5 + 3 * (grp < 4 ? grp : 4));
        }
    }
    SQ_TRACE_POINT(19);
}

// y[b, y_off + r] = row_scale[r] * sum over column slices (in slice order) of part[s, b, r]
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ part, int ks, int B, int R,
                                                            const uint16_t* __restrict__ row_scale, void* y, int64_t ldy,
                                                            int y_off, int y_dtype);

// op 0: launch; op 1: workgroups of `threads` threads and `smem` bytes of LDS that fit on one CU
template <int BITS, int D, int RW, int NT>
static inline int mma_inst(int op, const MmaArgs& a, int grid, int threads, size_t smem, hipStream_t s) {
    void (*k)(MmaArgs) = a.table_bytes ? rows_mfma_kernel<BITS, D, RW, NT, true> : rows_mfma_kernel<BITS, D, RW, NT, false>;
    if (op == 1) {
        static std::mutex mu;
        static std::unordered_map<uint64_t, int> cache;
        const uint64_t key = ((uint64_t)threads << 40) | ((uint64_t)(a.table_bytes != 0) << 39) | (uint64_t)smem;
        std::lock_guard<std::mutex> lock(mu);
        auto it = cache.find(key);
        if (it != cache.end()) return it->second;
        if (smem > 64 * 1024) {      // allow the 160 KB of a gfx950 CU
            (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipGetLastError();
        }
        hipFuncAttributes fa;
        int n = 1;
        if (hipFuncGetAttributes(&fa, (const void*)k) == hipSuccess && fa.numRegs > 0) {
            int wps = 512 / ((fa.numRegs + 7) / 8 * 8);     // 512 VGPRs per SIMD lane, granules of 8
            if (wps > 8) wps = 8;
            n = 4 * wps / (threads / 64);
        } else {
            (void)hipGetLastError();
        }
        if (smem && (size_t)n * smem > 160 * 1024) n = (int)(160 * 1024 / smem);
        if (n < 1) n = 1;
        cache[key] = n;
        return n;
    }
    hipLaunchKernelGGL(k, dim3(grid), dim3(threads), smem, s, a);
    return check_launch("sq_linear_small(mfma)");
}

// (RW, NT) pairs built per format: RW * SPU * NT <= 32 activation operands (128 registers) per lane
template <int BITS, int D>
static inline int mma_dispatch(int op, const MmaArgs& a, int RW, int NT, int grid, int threads, size_t smem, hipStream_t s) {
    constexpr int SPU = (unit_of<BITS>::UD * 32 / BITS) / (8 / D);
    constexpr int R1 = 32 / SPU;          // most rounds per wave with 16 activation rows
#define SQ_MMA(RW_, NT_) if (RW == RW_ && NT == NT_) return mma_inst<BITS, D, RW_, NT_>(op, a, grid, threads, smem, s)
    SQ_MMA(R1, 1);
    SQ_MMA(R1 / 2, 1);
    SQ_MMA(R1 / 2, 2);
    if constexpr (R1 >= 4) {
        SQ_MMA(R1 / 4, 1);
        SQ_MMA(R1 / 4, 2);
    }
#undef SQ_MMA
    return fail(SQ_EUNSUPPORTED, "sq_linear_small: no matrix-core kernel for %d rounds, %d token tiles", RW, NT);
}

#define SQ_MMA_FORMAT(BI, DD)                                                                               \
    int launch_mma_b##BI##d##DD(int op, const MmaArgs& a, int RW, int NT, int grid, int threads, size_t smem, \
                                hipStream_t s) {                                                            \
        return mma_dispatch<BI, DD>(op, a, RW, NT, grid, threads, smem, s);                                 \
    }

}  // namespace sq
