// Decode-time codebook product (B = 1..4 activation rows per pass) for gfx950.
//
// Work split.  A row's tag stream is cut into "units" of UD dwords holding TPU whole tags
// (16-bit tags: 4 dwords = 8 tags, one 128-bit load; 12-bit: 3 dwords = 8 tags; 8-bit: 4 dwords =
// 16 tags; 10-bit: 5 dwords = 16 tags).  A team of TS lanes owns a row at a time; lane tl of the
// team owns units tl, tl + TS, ... (S slots) of EVERY row the team visits, so the activations that
// multiply those units never change: they sit in registers as packed fp16 pairs for the whole
// kernel (bf16 activations are converted once, exactly for every fp16-normal value).  The only
// per-row traffic is the tag stream itself, read with one wide coalesced load per slot and
// prefetched one batch of rows ahead, plus one gather per tag from the codebook, which is
// staged in LDS when it fits and read through L1/L2 otherwise.  Products are v_dot2_f32_f16
// (fp16 x fp16 pairs, fp32 accumulate) with one accumulator per row in flight, so consecutive
// dot instructions are independent.  The team sum is six DPP adds (no LDS traffic); teams wider
// than a wave add their per-wave partials through LDS once per batch.
//
// Each team walks a contiguous range of row_order (rows sorted by column order), so the column
// order changes at most M - 1 times per matrix; a batch whose rows do not all share the
// current order takes a one-row-at-a-time path that reloads the activation registers from
// the pre-permuted copy xp[order].
#pragma once
#include <mutex>
#include <unordered_map>
#include "sq_common.h"

namespace sq {

constexpr int GEMV_MAX_PIECES = 4;
constexpr int GEMV_PF = 2;   // rows per batch; two batches of tag loads are in flight per lane

struct GemvPiece {
    sq_matrix m;
    const uint16_t* xp;   // fp16 [M, B, C] pre-permuted activations (pieces with column orders) or NULL
    int U;                // units per row
    int wg_begin;         // first workgroup of this piece
    int wg_count;         // workgroups that share this piece's rows
};

struct GemvArgs {
    GemvPiece p[GEMV_MAX_PIECES];
    int n;
    const uint16_t* x;
    int64_t ldx;
    void* y;
    int64_t ldy;
    int B, b0;            // this launch covers activation rows b0 .. b0 + NB - 1 (clipped to B)
    int x_dtype, y_dtype;
    int TS;               // team size: 16, 32, 64 or 64 * waves-per-row
    int table_bytes;      // bytes of codebook staged in LDS (0 = read through cache)
};

template <int BITS> struct unit_of;
template <> struct unit_of<16> { static constexpr int UD = 4; };
template <> struct unit_of<8> { static constexpr int UD = 4; };
template <> struct unit_of<12> { static constexpr int UD = 3; };
template <> struct unit_of<10> { static constexpr int UD = 5; };

template <int N> struct dwords { uint32_t v[N]; };

template <int UD>
__device__ __forceinline__ dwords<UD> load_unit(const uint32_t* __restrict__ p) {
    dwords<UD> r;
    if constexpr (UD == 4) {
        const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
        r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
    } else if constexpr (UD == 3) {
        const u32x3 t = __builtin_nontemporal_load(reinterpret_cast<const u32x3*>(p));
        r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z;
    } else {
#pragma unroll
        for (int i = 0; i < UD; ++i) r.v[i] = __builtin_nontemporal_load(p + i);
    }
    return r;
}

// Tag t of a unit, compile-time position.
template <int BITS, int UD>
__device__ __forceinline__ uint32_t unit_tag(const dwords<UD>& u, int t) {
    const int p = t * BITS, w = p >> 5, s = p & 31;
    uint32_t v;
    if (s + BITS <= 32) v = u.v[w] >> s;
    else v = __builtin_amdgcn_alignbit(u.v[w + 1 < UD ? w + 1 : w], u.v[w], s);
    return (s + BITS == 32) ? v : v & ((1u << BITS) - 1u);
}

// v + (v moved across lanes by a DPP pattern); lanes the pattern leaves out add zero
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
    const int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false);
    return v + __builtin_bit_cast(float, t);
}

// Sum over each team of `span` lanes (16, 32 or 64); valid in the LAST lane of every team.
__device__ __forceinline__ float team_sum(float v, int span) {
    v = dpp_add<0xB1, 0xf>(v);                     // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xf>(v);                     // quad_perm [2,3,0,1]
    v = dpp_add<0x141, 0xf>(v);                    // row_half_mirror
    v = dpp_add<0x140, 0xf>(v);                    // row_mirror: every lane holds its row-of-16 sum
    if (span >= 32) v = dpp_add<0x142, 0xa>(v);    // row_bcast15 into rows 1 and 3
    if (span >= 64) v = dpp_add<0x143, 0xc>(v);    // row_bcast31 into rows 2 and 3
    return v;
}

// Register estimate of one instantiation -> workgroup size limit the compiler may assume.
template <int BITS, int D, int S, int NB> struct gemv_cfg {
    static constexpr int UD = unit_of<BITS>::UD;
    static constexpr int TPU = UD * 32 / BITS;
    static constexpr int XH = TPU * D / 2;
    static constexpr int XW = NB * S * XH;            // dwords of activations a lane keeps in registers
    static constexpr bool OK = XW <= 192;
    static constexpr int LB = XW < 64 ? 512 : 256;    // threads per workgroup it is built for (256 or 512 VGPRs per lane)
};

template <int D> struct cw_t;
template <> struct cw_t<8> { typedef u32x4 type; };
template <> struct cw_t<4> { typedef u32x2 type; };

// Codebook into LDS, eight 16-byte loads in flight per thread before the first store.
__device__ __forceinline__ void stage_table(const uint16_t* table, int bytes, unsigned char* smem) {
    const u32x4* src = reinterpret_cast<const u32x4*>(table);
    u32x4* dst = reinterpret_cast<u32x4*>(smem);
    const int n = bytes / 16, tid = threadIdx.x, step = blockDim.x;
    for (int i0 = tid; i0 < n; i0 += 8 * step) {
        u32x4 v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int i = i0 + k * step;
            v[k] = src[i < n ? i : n - 1];
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int i = i0 + k * step;
            if (i < n) dst[i] = v[k];
        }
    }
}

template <int BITS, int D, int S, int NB, bool LDS_TAB>
struct GemvBody {
    static constexpr int UD = unit_of<BITS>::UD;
    static constexpr int TPU = UD * 32 / BITS;      // tags per unit
    static constexpr int XH = TPU * D / 2;          // fp16 pairs of activation per slot
    static constexpr int H = D / 2;                 // fp16 pairs per codeword
    typedef typename cw_t<D>::type CW;

    // activation registers of this lane for column order `rm` (16-byte loads; bf16 -> fp16 once)
    static __device__ __forceinline__ void load_x(uint32_t (&xr)[NB][S][XH], const GemvArgs& a, const GemvPiece& P,
                                                  int rm, int tl, int nb) {
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int s = 0; s < S; ++s) {
                // lanes past the row's end and activation rows past B load a valid address and keep zeros:
                // no branch around the loads, so they all issue back to back
                const int u = tl + s * a.TS;
                const bool ok = b < nb && u < P.U;
                const int c0 = (u < P.U ? u : P.U - 1) * (TPU * D);
                const int bb = a.b0 + (b < nb ? b : nb - 1);
                const uint16_t* src = P.xp ? P.xp + ((int64_t)rm * a.B + bb) * P.m.C + c0
                                           : a.x + (int64_t)bb * a.ldx + c0;
                const bool cvt = !P.xp && a.x_dtype == SQ_BF16;
                u32x4 v[XH / 4];
#pragma unroll
                for (int i = 0; i < XH / 4; ++i) v[i] = *reinterpret_cast<const u32x4*>(src + 8 * i);
#pragma unroll
                for (int i = 0; i < XH / 4; ++i) {
                    u32x4 w = v[i];
                    if (cvt) { w.x = bf2h_x2(w.x); w.y = bf2h_x2(w.y); w.z = bf2h_x2(w.z); w.w = bf2h_x2(w.w); }
                    xr[b][s][4 * i] = ok ? w.x : 0u; xr[b][s][4 * i + 1] = ok ? w.y : 0u;
                    xr[b][s][4 * i + 2] = ok ? w.z : 0u; xr[b][s][4 * i + 3] = ok ? w.w : 0u;
                }
            }
    }

    // NF rows at once: acc[f][b] = sum over this lane's units of <codeword, activations>.  A slot past the
    // row's end holds zero tags and zero activations; its sum is dropped so that codeword 0 (possibly
    // non-finite) never reaches rows that do not use it.
    template <int NF>
    static __device__ __forceinline__ void rows(float (&out)[NF][NB], const dwords<UD> (&tg)[NF][S],
                                                const uint32_t (&boff)[NF], const uint32_t (&xr)[NB][S][XH],
                                                const bool (&live)[S], const unsigned char* smem,
                                                const unsigned char* table) {
#pragma unroll
        for (int f = 0; f < NF; ++f)
#pragma unroll
            for (int b = 0; b < NB; ++b) out[f][b] = 0.f;
#pragma unroll
        for (int s = 0; s < S; ++s) {
            float acc[NF][NB];
#pragma unroll
            for (int f = 0; f < NF; ++f)
#pragma unroll
                for (int b = 0; b < NB; ++b) acc[f][b] = 0.f;
#pragma unroll
            for (int t = 0; t < TPU; ++t) {
                CW cw[NF];
#pragma unroll
                for (int f = 0; f < NF; ++f) {
                    const uint32_t tag = unit_tag<BITS, UD>(tg[f][s], t) + boff[f];
                    if (LDS_TAB) cw[f] = *reinterpret_cast<const CW*>(smem + tag * (D * 2));
                    else cw[f] = *reinterpret_cast<const CW*>(table + (size_t)tag * (D * 2));
                }
#pragma unroll
                for (int h = 0; h < H; ++h)
#pragma unroll
                    for (int f = 0; f < NF; ++f) {
                        const uint32_t cwh = cw[f][h];   // copy first: bit_cast straight from a vector element reads element 0
                        const half2v c2 = __builtin_bit_cast(half2v, cwh);
#pragma unroll
                        for (int b = 0; b < NB; ++b)
                            acc[f][b] = __builtin_amdgcn_fdot2(c2, __builtin_bit_cast(half2v, xr[b][s][t * H + h]), acc[f][b], false);
                    }
            }
#pragma unroll
            for (int f = 0; f < NF; ++f)
#pragma unroll
                for (int b = 0; b < NB; ++b) out[f][b] += live[s] ? acc[f][b] : 0.f;
        }
    }
};

template <int BITS, int D, int S, int NB, bool LDS_TAB>
__global__ __launch_bounds__((gemv_cfg<BITS, D, S, NB>::LB)) void gemv_kernel(GemvArgs a) {
    typedef GemvBody<BITS, D, S, NB, LDS_TAB> K;
    constexpr int UD = K::UD, XH = K::XH, PF = GEMV_PF;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    int pi = 0;
    while (pi + 1 < a.n && (int)blockIdx.x >= a.p[pi + 1].wg_begin) ++pi;
    const GemvPiece& P = a.p[pi];
    const sq_matrix& m = P.m;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int TS = a.TS;
    const int wpr = TS > 64 ? TS >> 6 : 1;             // waves per row
    const int span = TS < 64 ? TS : 64;                // lanes of one wave that share a row
    const int tl = TS > 64 ? (wave % wpr) * 64 + lane : lane & (TS - 1);
    const int grp = TS > 64 ? wave / wpr : wave * (64 / TS) + lane / TS;   // team of this lane
    const int ngrp = TS > 64 ? nwaves / wpr : nwaves * (64 / TS);
    const bool writer = (lane & (span - 1)) == span - 1;                   // holds the team sum after team_sum()

    float* part = reinterpret_cast<float*>(smem + a.table_bytes);          // [ngrp][PF][wpr][NB] per-wave partial sums
    if (LDS_TAB) {
        stage_table(m.table, a.table_bytes, smem);
        __syncthreads();
    }

    // rows of this workgroup: positions [p0, p1) of row_order, a contiguous share per team
    const int wg = blockIdx.x - P.wg_begin;
    const int p0 = (int)((int64_t)m.R * wg / P.wg_count), p1 = (int)((int64_t)m.R * (wg + 1) / P.wg_count);
    const int rpt = (p1 - p0 + ngrp - 1) / ngrp;                           // rows per team
    const int q0 = p0 + grp * rpt, q1 = q0 + rpt < p1 ? q0 + rpt : p1;
    const int nbatch = (rpt + PF - 1) / PF;                                // same trip count for every team

    const uint32_t* tags = reinterpret_cast<const uint32_t*>(m.tags);
    const int nb = a.B - a.b0 < NB ? a.B - a.b0 : NB;
    bool live[S];
#pragma unroll
    for (int s = 0; s < S; ++s) live[s] = tl + s * TS < P.U;
    uint32_t xr[NB][S][XH];
    int cur_mask = m.row_mask ? -1 : 0;
    if (!m.row_mask) K::load_x(xr, a, P, 0, tl, nb);

    // a batch: PF consecutive rows of this team, their tags, codebook offsets and column orders
    // (everything a batch needs from memory is loaded here, so nothing waits behind the next batch's prefetch)
    struct Batch { dwords<UD> tg[PF][S]; int row[PF]; uint32_t boff[PF]; int order[PF]; float scale[PF]; };
    Batch cur, nxt;
    auto fetch = [&](int q, Batch& bt) {
#pragma unroll
        for (int f = 0; f < PF; ++f) {
            const int pos = q + f;
            const int r = pos < q1 ? (m.row_order ? m.row_order[pos] : pos) : -1;
            bt.row[f] = r;
            bt.boff[f] = (r >= 0 && m.row_book) ? (uint32_t)m.row_book[r] << BITS : 0u;
            bt.order[f] = (r >= 0 && m.row_mask) ? (int)m.row_mask[r] : 0;
            bt.scale[f] = r >= 0 ? h2f(m.row_scale[r]) : 0.f;
#pragma unroll
            for (int s = 0; s < S; ++s) {
                const int u = tl + s * TS;
                if (r >= 0 && u < P.U) bt.tg[f][s] = load_unit<UD>(tags + (int64_t)r * m.W + u * UD);
                else {
#pragma unroll
                    for (int i = 0; i < UD; ++i) bt.tg[f][s].v[i] = 0u;
                }
            }
        }
    };
    fetch(q0, cur);

    for (int it = 0; it < nbatch; ++it) {
        if (it + 1 < nbatch) fetch(q0 + (it + 1) * PF, nxt);
        float acc[PF][NB];
#pragma unroll
        for (int f = 0; f < PF; ++f)
#pragma unroll
            for (int b = 0; b < NB; ++b) acc[f][b] = 0.f;
        // One pass per distinct column order among the batch's rows: a single pass unless the batch
        // straddles an order boundary (at most M - 1 such batches per team walk).
        uint32_t pending = 0;
#pragma unroll
        for (int f = 0; f < PF; ++f) pending |= (cur.row[f] >= 0 ? 1u : 0u) << f;
        while (pending) {
            if (m.row_mask) {
                int want = cur_mask;
#pragma unroll
                for (int f = PF - 1; f >= 0; --f)
                    if (pending >> f & 1u) want = cur.order[f];                 // order of the first pending row
                if (want != cur_mask) { cur_mask = want; K::load_x(xr, a, P, want, tl, nb); }
            }
            float tmp[PF][NB];
            K::template rows<PF>(tmp, cur.tg, cur.boff, xr, live, smem, reinterpret_cast<const unsigned char*>(m.table));
#pragma unroll
            for (int f = 0; f < PF; ++f)
                if ((pending >> f & 1u) && cur.order[f] == cur_mask) {
#pragma unroll
                    for (int b = 0; b < NB; ++b) acc[f][b] = tmp[f][b];
                    pending &= ~(1u << f);
                }
        }
#pragma unroll
        for (int f = 0; f < PF; ++f)
#pragma unroll
            for (int b = 0; b < NB; ++b) acc[f][b] = team_sum(acc[f][b], span);
        if (wpr == 1) {
            if (writer) {
#pragma unroll
                for (int f = 0; f < PF; ++f) {
                    const int r = cur.row[f];
                    if (r < 0) continue;
                    const float sc = cur.scale[f];
                    for (int b = 0; b < nb; ++b)
                        store_y(a.y, a.y_dtype, (int64_t)(a.b0 + b) * a.ldy + m.y_off + r, acc[f][b] * sc);
                }
            }
        } else {
            if (lane == 63) {
#pragma unroll
                for (int f = 0; f < PF; ++f)
#pragma unroll
                    for (int b = 0; b < NB; ++b) part[((grp * PF + f) * wpr + wave % wpr) * NB + b] = acc[f][b];
            }
            __syncthreads();
            for (int i = tid; i < ngrp * PF * nb; i += blockDim.x) {
                const int b = i % nb, q = i / nb;                           // q = team * PF + f
                const int g = q / PF, f = q - g * PF;
                const int pos = p0 + g * rpt + it * PF + f;
                const int pend = p0 + (g + 1) * rpt < p1 ? p0 + (g + 1) * rpt : p1;
                if (pos < pend) {
                    const int r = m.row_order ? m.row_order[pos] : pos;
                    float v = 0.f;
                    for (int w = 0; w < wpr; ++w) v += part[(q * wpr + w) * NB + b];
                    store_y(a.y, a.y_dtype, (int64_t)(a.b0 + b) * a.ldy + m.y_off + r, v * h2f(m.row_scale[r]));
                }
            }
            __syncthreads();
        }
        cur = nxt;
    }
}

// Rows as wide as a wave or wider (TS = 64 * waves-per-row): the row a wave works on is uniform, so the
// row index, its base address, codebook offset and column order live in scalar registers and the inner
// loop is branch-free: lanes past the row's end re-read the last unit (their activations are zero and
// their sums are dropped), batches past the team's last row re-read it and skip the store.
template <int BITS, int D, int S, int NB, bool LDS_TAB>
__global__ __launch_bounds__((gemv_cfg<BITS, D, S, NB>::LB)) void gemv_wave_kernel(GemvArgs a) {
    typedef GemvBody<BITS, D, S, NB, LDS_TAB> K;
    constexpr int UD = K::UD, XH = K::XH, PF = GEMV_PF;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), nwaves = blockDim.x >> 6;
    int pi = 0;
    while (pi + 1 < a.n && (int)blockIdx.x >= a.p[pi + 1].wg_begin) ++pi;
    const GemvPiece& P = a.p[pi];
    const sq_matrix& m = P.m;
    const int TS = a.TS, wpr = TS >> 6;
    const int team = wave / wpr, wcol = wave - team * wpr, nteams = nwaves / wpr;
    const int tl = wcol * 64 + lane;

    float* part = reinterpret_cast<float*>(smem + a.table_bytes);          // [nteams][PF][wpr][NB] per-wave partial sums

    const int wg = blockIdx.x - P.wg_begin;
    const int p0 = (int)((int64_t)m.R * wg / P.wg_count), p1 = (int)((int64_t)m.R * (wg + 1) / P.wg_count);
    const int rpt = (p1 - p0 + nteams - 1) / nteams;                       // rows per team
    const int q0 = p0 + team * rpt, q1 = q0 + rpt < p1 ? q0 + rpt : p1;
    const int nbatch = (rpt + PF - 1) / PF;                                // same trip count for every team
    const bool has = q0 < q1;

    const uint32_t* tags = reinterpret_cast<const uint32_t*>(m.tags);
    const unsigned char* table = reinterpret_cast<const unsigned char*>(m.table);
    const int nb = a.B - a.b0 < NB ? a.B - a.b0 : NB;
    bool live[S];
    uint32_t uoff[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
        const int u = tl + s * TS;
        live[s] = u < P.U;
        uoff[s] = (uint32_t)(live[s] ? u : P.U - 1) * UD;
    }
    uint32_t xr[NB][S][XH];
    int cur_order = m.row_mask ? -1 : 0;
    if (!m.row_mask) K::load_x(xr, a, P, 0, tl, nb);

    // Row metadata (row id, scale, codebook offset, column order) of 64 consecutive positions is held one
    // position per lane and handed out with v_readlane, so the batch loop issues no global load besides the
    // tag stream and never waits behind its own prefetch.  Positions past the team's end repeat its last row.
    int cb = q0, mrow = 0, mord = 0;
    float mscale = 0.f;
    uint32_t mboff = 0u;
    auto refill = [&](int base) {
        cb = base;
        const int pos = base + lane < q1 ? base + lane : q1 - 1;
        mrow = m.row_order ? m.row_order[pos] : pos;
        mscale = h2f(m.row_scale[mrow]);
        mboff = m.row_book ? (uint32_t)m.row_book[mrow] << BITS : 0u;
        mord = m.row_mask ? (int)m.row_mask[mrow] : 0;
    };
    struct Batch { dwords<UD> t[PF][S]; int row[PF]; float scale[PF]; uint32_t boff[PF]; int order[PF]; };
    auto fetch = [&](int q, Batch& B) {
        if (q + PF > cb + 64) refill(q);
#pragma unroll
        for (int f = 0; f < PF; ++f) {
            const int pos = q + f < q1 ? q + f : q1 - 1;
            const int j = pos - cb;
            const int r = __builtin_amdgcn_readlane(mrow, j);
            B.row[f] = r;
            B.scale[f] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mscale), j));
            B.boff[f] = (uint32_t)__builtin_amdgcn_readlane((int)mboff, j);
            B.order[f] = __builtin_amdgcn_readlane(mord, j);
            const uint32_t* rp = tags + (size_t)r * m.W;
#pragma unroll
            for (int s = 0; s < S; ++s) B.t[f][s] = load_unit<UD>(rp + uoff[s]);
        }
    };

    auto process = [&](int it, const Batch& B) {
        float acc[PF][NB];
        if (has) {
            bool same = true;
#pragma unroll
            for (int f = 0; f < PF; ++f) same = same && B.order[f] == cur_order;
            if (same) {
                K::template rows<PF>(acc, B.t, B.boff, xr, live, smem, table);
            } else {
                // the column order changes inside this batch (at most M - 1 times per team): row by row
#pragma unroll
                for (int f = 0; f < PF; ++f) {
                    if (B.order[f] != cur_order) { cur_order = B.order[f]; K::load_x(xr, a, P, cur_order, tl, nb); }
                    float a1[1][NB];
                    const dwords<UD> (&t1)[1][S] = reinterpret_cast<const dwords<UD> (&)[1][S]>(B.t[f]);
                    const uint32_t b1[1] = {B.boff[f]};
                    K::template rows<1>(a1, t1, b1, xr, live, smem, table);
#pragma unroll
                    for (int b = 0; b < NB; ++b) acc[f][b] = a1[0][b];
                }
            }
#pragma unroll
            for (int f = 0; f < PF; ++f)
#pragma unroll
                for (int b = 0; b < NB; ++b) acc[f][b] = team_sum(acc[f][b], 64);
        }
        const int qb = q0 + it * PF;
        if (wpr == 1) {
            if (has && lane == 63) {
#pragma unroll
                for (int f = 0; f < PF; ++f) {
                    if (qb + f >= q1) continue;
                    for (int b = 0; b < nb; ++b)
                        store_y(a.y, a.y_dtype, (int64_t)(a.b0 + b) * a.ldy + m.y_off + B.row[f], acc[f][b] * B.scale[f]);
                }
            }
        } else {
            if (has && lane == 63) {
#pragma unroll
                for (int f = 0; f < PF; ++f)
#pragma unroll
                    for (int b = 0; b < NB; ++b) part[((team * PF + f) * wpr + wcol) * NB + b] = acc[f][b];
            }
            __syncthreads();
            // the first wave of each team adds the team's per-wave partials (lane = f * NB + b)
            if (has && wcol == 0 && lane < PF * NB) {
                const int f = lane / NB, b = lane - f * NB;
                if (qb + f < q1 && b < nb) {
                    float v = 0.f;
                    for (int w = 0; w < wpr; ++w) v += part[((team * PF + f) * wpr + w) * NB + b];
                    int r = B.row[0];
                    float sc = B.scale[0];
#pragma unroll
                    for (int g = 1; g < PF; ++g)
                        if (f == g) { r = B.row[g]; sc = B.scale[g]; }
                    store_y(a.y, a.y_dtype, (int64_t)(a.b0 + b) * a.ldy + m.y_off + r, v * sc);
                }
            }
            __syncthreads();
        }
    };

    // start-up: metadata, activations and codebook are requested together and the first tag fetch follows
    // as soon as the row ids are known, so the kernel pays two memory latencies before its first product
    Batch bA, bB;
    if (has) refill(q0);
    if (LDS_TAB) stage_table(m.table, a.table_bytes, smem);
    if (has) fetch(q0, bA);
    if (LDS_TAB) __syncthreads();
    for (int it = 0; it < nbatch; it += 2) {                               // two batches per trip: A computes while B loads
        if (has && it + 1 < nbatch) fetch(q0 + (it + 1) * PF, bB);
        process(it, bA);
        if (it + 1 < nbatch) {
            if (has && it + 2 < nbatch) fetch(q0 + (it + 2) * PF, bA);
            process(it + 1, bB);
        }
    }
}

// Workgroups of `threads` threads and `smem` bytes of LDS that fit on one CU (from the runtime's occupancy
// calculator, i.e. from the registers the compiler really used); cached per instantiation.
template <int BITS, int D, int S, int NB, bool LDS_TAB, bool WAVE>
static inline int occupancy_of(int threads, size_t smem) {
    static std::mutex mu;
    static std::unordered_map<uint64_t, int> cache;
    const uint64_t key = ((uint64_t)threads << 32) | (uint64_t)smem;
    std::lock_guard<std::mutex> lock(mu);
    auto it = cache.find(key);
    if (it != cache.end()) return it->second;
    void (*k)(GemvArgs) = WAVE ? gemv_wave_kernel<BITS, D, S, NB, LDS_TAB> : gemv_kernel<BITS, D, S, NB, LDS_TAB>;
    if (smem > 64 * 1024) {      // allow the 160 KB of a gfx950 CU
        (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        (void)hipGetLastError();
    }
    // from the registers the compiler used: 512 VGPRs per SIMD lane in granules of 8, at most 8 waves per SIMD
    hipFuncAttributes fa;
    int n = 1;
    if (hipFuncGetAttributes(&fa, (const void*)k) == hipSuccess && fa.numRegs > 0) {
        int wps = 512 / ((fa.numRegs + 7) / 8 * 8);
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

// op 0: launch; op 1: return the occupancy (workgroups per CU) for (threads, smem)
template <int BITS, int D, int S, int NB>
static inline int launch_inst(int op, const GemvArgs& a, int grid, int threads, size_t smem, hipStream_t s) {
    if constexpr (!gemv_cfg<BITS, D, S, NB>::OK) {
        return fail(SQ_EUNSUPPORTED, "sq_linear_small: no kernel for bits %d d %d slots %d rows %d", BITS, D, S, NB);
    } else {
        if (threads > gemv_cfg<BITS, D, S, NB>::LB)
            return fail(SQ_ELAUNCH, "sq_linear_small: %d threads > %d", threads, gemv_cfg<BITS, D, S, NB>::LB);
        const bool wave = a.TS >= 64;
        if (op == 1) {
            if (wave) return a.table_bytes ? occupancy_of<BITS, D, S, NB, true, true>(threads, smem)
                                           : occupancy_of<BITS, D, S, NB, false, true>(threads, smem);
            return a.table_bytes ? occupancy_of<BITS, D, S, NB, true, false>(threads, smem)
                                 : occupancy_of<BITS, D, S, NB, false, false>(threads, smem);
        }
        void (*k)(GemvArgs);
        if (wave) k = a.table_bytes ? gemv_wave_kernel<BITS, D, S, NB, true> : gemv_wave_kernel<BITS, D, S, NB, false>;
        else k = a.table_bytes ? gemv_kernel<BITS, D, S, NB, true> : gemv_kernel<BITS, D, S, NB, false>;
        hipLaunchKernelGGL(k, dim3(grid), dim3(threads), smem, s, a);
        return check_launch("sq_linear_small");
    }
}

template <int BITS, int D, int S>
static inline int launch_nb(int op, const GemvArgs& a, int nbt, int grid, int threads, size_t smem, hipStream_t s) {
    switch (nbt) {
        case 1: return launch_inst<BITS, D, S, 1>(op, a, grid, threads, smem, s);
        case 2: return launch_inst<BITS, D, S, 2>(op, a, grid, threads, smem, s);
        default: return launch_inst<BITS, D, S, 4>(op, a, grid, threads, smem, s);
    }
}

template <int BITS, int D>
static inline int launch_s(int op, const GemvArgs& a, int S, int nbt, int grid, int threads, size_t smem, hipStream_t s) {
    switch (S) {
        case 1: return launch_nb<BITS, D, 1>(op, a, nbt, grid, threads, smem, s);
        case 2: return launch_nb<BITS, D, 2>(op, a, nbt, grid, threads, smem, s);
        case 3: return launch_nb<BITS, D, 3>(op, a, nbt, grid, threads, smem, s);
        case 5: return launch_nb<BITS, D, 5>(op, a, nbt, grid, threads, smem, s);
    }
    return fail(SQ_EUNSUPPORTED, "sq_linear_small: slots %d", S);
}

// One translation unit per tag format instantiates its kernels behind a plain function.
#define SQ_GEMV_FORMAT(BI, DD)                                                                                  \
    int launch_gemv_b##BI##d##DD(int op, const GemvArgs& a, int S, int nbt, int grid, int threads, size_t smem, \
                                 hipStream_t s) {                                                              \
        return launch_s<BI, DD>(op, a, S, nbt, grid, threads, smem, s);                                        \
    }

}  // namespace sq
