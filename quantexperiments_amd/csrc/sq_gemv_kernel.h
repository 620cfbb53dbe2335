// Decode-time codebook product (B = 1..4 activation rows per pass) for gfx950.
//
// Work split.  A row's tag stream is cut into "units" of UD dwords holding TPU whole tags
// (16-bit tags: 4 dwords = 8 tags, one 128-bit load; 12-bit: 3 dwords = 8 tags; 8-bit: 4 dwords =
// 16 tags; 10-bit: 5 dwords = 16 tags).  A team of TS lanes owns a row at a time; lane tl of the
// team owns units tl, tl + TS, ... (S slots) of EVERY row the team visits, so the activations that
// multiply those units never change: they sit in registers as packed fp16 pairs for the whole
// kernel (bf16 activations are converted once, exactly for every fp16-normal value).  The only
// per-row traffic is the tag stream itself, read with one wide coalesced load per slot, plus
// one gather per tag from the codebook, which is staged in LDS when it fits and read through
// L1/L2 otherwise.  Products are v_dot2_f32_f16 (fp16 x fp16 pairs, fp32 accumulate); the team
// sum is a cross-lane butterfly, and teams wider than a wave add their per-wave partials
// through LDS once per row block.
//
// Column orders: rows are visited in row_order (sorted by mask), a lane reloads its activation
// registers from the pre-permuted copy xp[mask] only when the mask of its row changes.
#pragma once
#include "sq_common.h"

namespace sq {

constexpr int GEMV_MAX_PIECES = 4;
constexpr int GEMV_PF = 4;   // rows whose tag loads are issued before any of them is consumed

struct GemvPiece {
    sq_matrix m;
    const uint16_t* xp;   // fp16 [M, B, C] pre-permuted activations (M > 1) or NULL
    int U;                // units per row
    int wg_begin;         // first workgroup of this piece
    int wg_count;
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
    return v & ((1u << BITS) - 1u);
}

// Register estimate of one instantiation -> workgroup size limit the compiler may assume.
template <int BITS, int D, int S, int NB> struct gemv_cfg {
    static constexpr int UD = unit_of<BITS>::UD;
    static constexpr int TPU = UD * 32 / BITS;
    static constexpr int XH = TPU * D / 2;
    static constexpr int REGS = NB * S * XH + GEMV_PF * S * UD + 56;
    static constexpr bool OK = REGS <= 440;
    static constexpr int LB = REGS <= 256 ? 512 : 256;      // threads per workgroup the kernel is built for
};

template <int D> struct cw_t;
template <> struct cw_t<8> { typedef u32x4 type; };
template <> struct cw_t<4> { typedef u32x2 type; };

template <int BITS, int D, int S, int NB, bool LDS_TAB>
__global__ __launch_bounds__((gemv_cfg<BITS, D, S, NB>::LB)) void gemv_kernel(GemvArgs a) {
    constexpr int UD = unit_of<BITS>::UD;
    constexpr int TPU = UD * 32 / BITS;      // tags per unit
    constexpr int XH = TPU * D / 2;          // fp16 pairs of activation per slot
    constexpr int H = D / 2;                 // fp16 pairs per codeword
    typedef typename cw_t<D>::type CW;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    int pi = 0;
    while (pi + 1 < a.n && (int)blockIdx.x >= a.p[pi + 1].wg_begin) ++pi;
    const GemvPiece& P = a.p[pi];
    const sq_matrix& m = P.m;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int TS = a.TS;
    const int wpr = TS > 64 ? TS >> 6 : 1;             // waves per row
    const int rpw = TS < 64 ? 64 / TS : 1;             // rows per wave
    const int tl = TS > 64 ? (wave % wpr) * 64 + lane : lane & (TS - 1);
    const int grp = TS > 64 ? wave / wpr : wave * rpw + lane / TS;   // row group of this lane
    const int ngrp = TS > 64 ? nwaves / wpr : nwaves * rpw;

    // ---- codebook into LDS
    float* part = reinterpret_cast<float*>(smem + a.table_bytes);      // [GEMV_PF * ngrp rows][wpr][NB] per-wave partial sums
    if (LDS_TAB) {
        const u32x4* src = reinterpret_cast<const u32x4*>(m.table);
        u32x4* dst = reinterpret_cast<u32x4*>(smem);
        for (int i = tid; i < a.table_bytes / 16; i += blockDim.x) dst[i] = src[i];
        __syncthreads();
    }

    // ---- rows of this workgroup: positions [p0, p1) of row_order
    const int wg = blockIdx.x - P.wg_begin;
    const int p0 = (int)((int64_t)m.R * wg / P.wg_count), p1 = (int)((int64_t)m.R * (wg + 1) / P.wg_count);

    uint32_t xr[NB][S][XH];
    int cur_mask = -1;
    const uint32_t* tags = reinterpret_cast<const uint32_t*>(m.tags);
    const int nb = a.B - a.b0 < NB ? a.B - a.b0 : NB;

    for (int pbase = p0; pbase < p1; pbase += ngrp * GEMV_PF) {
        dwords<UD> tg[GEMV_PF][S];
        int rows[GEMV_PF];
#pragma unroll
        for (int f = 0; f < GEMV_PF; ++f) {
            const int pos = pbase + f * ngrp + grp;
            rows[f] = pos < p1 ? (m.row_order ? m.row_order[pos] : pos) : -1;
#pragma unroll
            for (int s = 0; s < S; ++s) {
                const int u = tl + s * TS;
                if (rows[f] >= 0 && u < P.U) tg[f][s] = load_unit<UD>(tags + (int64_t)rows[f] * m.W + u * UD);
                else {
#pragma unroll
                    for (int i = 0; i < UD; ++i) tg[f][s].v[i] = 0u;
                }
            }
        }
#pragma unroll
        for (int f = 0; f < GEMV_PF; ++f) {
            const int r = rows[f];
            const int rm = (r >= 0 && m.row_mask) ? m.row_mask[r] : 0;
            if (r >= 0 && rm != cur_mask) {          // (re)load the activation registers
                cur_mask = rm;
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int s = 0; s < S; ++s) {
                        const int u = tl + s * TS;
                        const bool ok = b < nb && u < P.U;
                        const int c0 = u * (TPU * D);
                        if (P.xp) {
                            const uint32_t* src = reinterpret_cast<const uint32_t*>(
                                P.xp + ((int64_t)rm * a.B + a.b0 + b) * m.C + c0);
#pragma unroll
                            for (int i = 0; i < XH; ++i) xr[b][s][i] = ok ? src[i] : 0u;
                        } else {
                            const uint32_t* src = reinterpret_cast<const uint32_t*>(a.x + (int64_t)(a.b0 + b) * a.ldx + c0);
#pragma unroll
                            for (int i = 0; i < XH; ++i) {
                                const uint32_t v = ok ? src[i] : 0u;
                                xr[b][s][i] = a.x_dtype == SQ_BF16 ? bf2h_x2(v) : v;
                            }
                        }
                    }
            }
            float acc[NB];
#pragma unroll
            for (int b = 0; b < NB; ++b) acc[b] = 0.f;
            const uint32_t boff = (r >= 0 && m.row_book) ? (uint32_t)m.row_book[r] << BITS : 0u;
#pragma unroll
            for (int s = 0; s < S; ++s) {
                float sl[NB];        // this slot's sum; dropped for lanes past the row's end so that
#pragma unroll                       // codeword 0 (what their zero tags gather) never reaches the result
                for (int b = 0; b < NB; ++b) sl[b] = 0.f;
#pragma unroll
                for (int t = 0; t < TPU; ++t) {
                    const uint32_t tag = unit_tag<BITS, UD>(tg[f][s], t) + boff;
                    CW cw;
                    if (LDS_TAB) cw = *reinterpret_cast<const CW*>(smem + tag * (D * 2));
                    else cw = *reinterpret_cast<const CW*>(reinterpret_cast<const unsigned char*>(m.table) + (size_t)tag * (D * 2));
#pragma unroll
                    for (int h = 0; h < H; ++h) {
                        const uint32_t cwh = cw[h];      // copy first: bit_cast straight from a vector element reads element 0
                        const half2v c2 = __builtin_bit_cast(half2v, cwh);
#pragma unroll
                        for (int b = 0; b < NB; ++b)
                            sl[b] = __builtin_amdgcn_fdot2(c2, __builtin_bit_cast(half2v, xr[b][s][t * H + h]), sl[b], false);
                    }
                }
                const bool live = tl + s * TS < P.U;
#pragma unroll
                for (int b = 0; b < NB; ++b) acc[b] += live ? sl[b] : 0.f;
            }
            // ---- team sum
            const int span = TS < 64 ? TS : 64;
#pragma unroll
            for (int b = 0; b < NB; ++b)
                for (int o = span >> 1; o > 0; o >>= 1) acc[b] += __shfl_xor(acc[b], o, 64);
            if (wpr == 1) {
                if ((lane & (span - 1)) == 0 && r >= 0) {
                    const float sc = h2f(m.row_scale[r]);
                    for (int b = 0; b < nb; ++b) {
                        const int64_t o = (int64_t)(a.b0 + b) * a.ldy + m.y_off + r;
                        const float v = acc[b] * sc;
                        if (a.y_dtype == SQ_BF16) reinterpret_cast<uint16_t*>(a.y)[o] = f2bf(v);
                        else if (a.y_dtype == SQ_F16) reinterpret_cast<uint16_t*>(a.y)[o] = f2h(v);
                        else reinterpret_cast<float*>(a.y)[o] = v;
                    }
                }
            } else if (lane == 0) {
                // part[(f * ngrp + grp) * wpr + wave % wpr][b]
#pragma unroll
                for (int b = 0; b < NB; ++b) part[(((f * ngrp + grp) * wpr) + wave % wpr) * NB + b] = acc[b];
            }
        }
        if (wpr > 1) {
            __syncthreads();
            for (int i = tid; i < GEMV_PF * ngrp * nb; i += blockDim.x) {
                const int b = i % nb, q = i / nb;              // q = f * ngrp + grp
                const int pos = pbase + q;
                if (pos < p1) {
                    const int r = m.row_order ? m.row_order[pos] : pos;
                    float v = 0.f;
                    for (int w = 0; w < wpr; ++w) v += part[(q * wpr + w) * NB + b];
                    v *= h2f(m.row_scale[r]);
                    const int64_t o = (int64_t)(a.b0 + b) * a.ldy + m.y_off + r;
                    if (a.y_dtype == SQ_BF16) reinterpret_cast<uint16_t*>(a.y)[o] = f2bf(v);
                    else if (a.y_dtype == SQ_F16) reinterpret_cast<uint16_t*>(a.y)[o] = f2h(v);
                    else reinterpret_cast<float*>(a.y)[o] = v;
                }
            }
            __syncthreads();
        }
    }
}

template <int BITS, int D, int S, int NB>
static inline int launch_inst(const GemvArgs& a, int grid, int threads, size_t smem, hipStream_t s) {
    if constexpr (!gemv_cfg<BITS, D, S, NB>::OK) {
        return fail(SQ_EUNSUPPORTED, "sq_linear_small: no kernel for bits %d d %d slots %d rows %d", BITS, D, S, NB);
    } else {
        if (threads > gemv_cfg<BITS, D, S, NB>::LB)
            return fail(SQ_ELAUNCH, "sq_linear_small: %d threads > %d", threads, gemv_cfg<BITS, D, S, NB>::LB);
        if (a.table_bytes) {
            auto k = gemv_kernel<BITS, D, S, NB, true>;
            if (smem > 64 * 1024) {
                static bool raised = false;
                if (!raised) {
                    (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
                    (void)hipGetLastError();
                    raised = true;
                }
            }
            hipLaunchKernelGGL(k, dim3(grid), dim3(threads), smem, s, a);
        } else {
            hipLaunchKernelGGL((gemv_kernel<BITS, D, S, NB, false>), dim3(grid), dim3(threads), smem, s, a);
        }
        return check_launch("sq_linear_small");
    }
}

template <int BITS, int D, int S>
static inline int launch_nb(const GemvArgs& a, int nbt, int grid, int threads, size_t smem, hipStream_t s) {
    switch (nbt) {
        case 1: return launch_inst<BITS, D, S, 1>(a, grid, threads, smem, s);
        case 2: return launch_inst<BITS, D, S, 2>(a, grid, threads, smem, s);
        default: return launch_inst<BITS, D, S, 4>(a, grid, threads, smem, s);
    }
}

template <int BITS, int D>
static inline int launch_s(const GemvArgs& a, int S, int nbt, int grid, int threads, size_t smem, hipStream_t s) {
    switch (S) {
        case 1: return launch_nb<BITS, D, 1>(a, nbt, grid, threads, smem, s);
        case 2: return launch_nb<BITS, D, 2>(a, nbt, grid, threads, smem, s);
        case 3: return launch_nb<BITS, D, 3>(a, nbt, grid, threads, smem, s);
        case 5: return launch_nb<BITS, D, 5>(a, nbt, grid, threads, smem, s);
    }
    return fail(SQ_EUNSUPPORTED, "sq_linear_small: slots %d", S);
}

// One translation unit per tag format instantiates its kernels behind a plain function.
#define SQ_GEMV_FORMAT(BI, DD)                                                                              \
    int launch_gemv_b##BI##d##DD(const GemvArgs& a, int S, int nbt, int grid, int threads, size_t smem,   \
                                 hipStream_t s) {                                                          \
        return launch_s<BI, DD>(a, S, nbt, grid, threads, smem, s);                                        \
    }

}  // namespace sq
