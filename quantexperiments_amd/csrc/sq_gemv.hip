// Host side of the decode-time product: picks the team geometry per shape, fuses stacked pieces
// into one persistent launch, prepares permuted activations for pieces with column orders.
#include "sq_rows_mfma.h"
#include "sq_stream.h"

namespace sq {

int launch_gemv_b16d8(int, const GemvArgs&, int, int, int, int, size_t, hipStream_t);
int launch_gemv_b12d4(int, const GemvArgs&, int, int, int, int, size_t, hipStream_t);
int launch_gemv_b10d4(int, const GemvArgs&, int, int, int, int, size_t, hipStream_t);
int launch_gemv_b8d4(int, const GemvArgs&, int, int, int, int, size_t, hipStream_t);
int launch_mma_b16d8(int, const MmaArgs&, int, int, int, int, size_t, hipStream_t);
int launch_mma_b12d4(int, const MmaArgs&, int, int, int, int, size_t, hipStream_t);
int launch_mma_b10d4(int, const MmaArgs&, int, int, int, int, size_t, hipStream_t);
int launch_mma_b8d4(int, const MmaArgs&, int, int, int, int, size_t, hipStream_t);

__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ part, int ks, int B, int R,
                                                            const uint16_t* __restrict__ row_scale, void* y, int64_t ldy,
                                                            int y_off, int y_dtype) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= B * R) return;
    const int b = i / R, r = i - b * R;
    float v = 0.f;
    for (int s = 0; s < ks; ++s) v += part[((int64_t)s * B + b) * R + r];
    store_y(y, y_dtype, (int64_t)b * ldy + y_off + r, v * h2f(row_scale[r]));
}

// xp[m, b, c] = fp16(x[b, perms[m, c]])
__global__ __launch_bounds__(256) void permute_x_kernel(const uint16_t* __restrict__ x, int64_t ldx, int x_dtype,
                                                        const int32_t* __restrict__ perms, int M, int B, int C,
                                                        uint16_t* __restrict__ xp) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)M * B * C) return;
    const int c = (int)(i % C);
    const int b = (int)((i / C) % B);
    const int mk = (int)(i / ((int64_t)C * B));
    const uint16_t v = x[(int64_t)b * ldx + perms[(int64_t)mk * C + c]];
    xp[i] = x_dtype == SQ_BF16 ? __builtin_bit_cast(uint16_t, bf2h(v)) : v;
}

// ------------------------------------------------------------------------------------------ host

int launch_small_generic(const sq_matrix* mats, int n, const void* x, int x_dtype, int64_t ldx, void* y,
                         int y_dtype, int64_t ldy, int B, hipStream_t s);

static int unit_dwords(int bits) { return bits == 12 ? 3 : bits == 10 ? 5 : 4; }

static bool fast_shape(const sq_matrix& m) {
    if (!m.tags) return false;                                   // held as its tag stream only
    const bool fmt = (m.d == 8 && m.bits == 16) || (m.d == 4 && (m.bits == 12 || m.bits == 10 || m.bits == 8));
    if (!fmt) return false;
    if (m.W % unit_dwords(m.bits)) return false;                 // rows must be whole units
    if (((uintptr_t)m.tags & 15) || ((uintptr_t)m.table & 15)) return false;
    if ((int64_t)(m.C / m.d) * m.bits != (int64_t)m.W * 32) return false;   // no pad bits inside the last unit
    return true;
}

// ---- tile-major copy of the tags for the matrix-core decode kernel (d = 4 formats, whose codebooks live in
// LDS and which have no slice stream).  In the file's row-major layout the 16 lanes of a quarter wave read 16
// different rows, 48 bytes each; in the copy the units of a 16-row tile are stored unit by unit,
//     tiled[((t * U + u) * 16 + i) * UD + w] = tags[(16 t + i) * W + u * UD + w]      (rows past R: zeros)
// so the same 16 lanes read 16 * UD consecutive dwords and a wave load covers one contiguous piece.
bool tiled_format_ok(int R, int W, int C, int d, int bits) {
    if (!(d == 4 && (bits == 12 || bits == 10 || bits == 8))) return false;
    if (R <= 0 || C % d || W % unit_dwords(bits)) return false;
    return (int64_t)(C / d) * bits == (int64_t)W * 32;
}

size_t tiled_bytes(int R, int W) { return (size_t)((R + 15) / 16) * 16 * W * 4; }

void tiled_build(const uint32_t* tags, int R, int W, int bits, uint32_t* out) {
    const int ud = unit_dwords(bits), U = W / ud, ntiles = (R + 15) / 16;
    for (int t = 0; t < ntiles; ++t)
        for (int u = 0; u < U; ++u)
            for (int i = 0; i < 16; ++i) {
                uint32_t* dst = out + (((size_t)t * U + u) * 16 + i) * ud;
                const int r = t * 16 + i;
                for (int w = 0; w < ud; ++w) dst[w] = r < R ? tags[(size_t)r * W + u * ud + w] : 0u;
            }
}

static size_t xp_bytes(const sq_matrix& m, int B) {
    return (((size_t)(m.M > 1 ? m.M : 1) * B * m.C * 2) + 255) & ~(size_t)255;
}

struct Plan { int TS, S, nwaves; };

// Host mirror of gemv_cfg<>::XW / OK / LB.
static int cfg_xw(int bits, int d, int S, int NB) {
    const int ud = unit_dwords(bits);
    return NB * S * (ud * 32 / bits * d / 2);
}
static int cfg_lb(int bits, int d, int S, int NB) { return cfg_xw(bits, d, S, NB) < 64 ? 512 : 256; }

// Team size / slots for U units per row: fewest idle lanes, then fewest slots.
static Plan plan_for(int U, int bits, int d) {
    Plan best{0, 0, 0};
    double best_eff = -1.0;
    const int cands[] = {16, 32, 64, 128, 192, 256, 320, 384, 448, 512, 640, 768, 1024};
    const int slots[] = {1, 2, 3, 5};
    for (int ts : cands)
        for (int s : slots) {
            if (ts * s < U) continue;
            if (cfg_xw(bits, d, s, 1) > 192) break;
            if (ts > cfg_lb(bits, d, s, 1)) break;
            const double eff = (double)U / (ts * s) - 0.02 * (s - 1) - (ts > 64 ? 0.05 : 0.0);   // barriers cost
            if (eff > best_eff + 1e-9) { best_eff = eff; best.TS = ts; best.S = s; }
            break;
        }
    if (best.TS == 0) return best;
    // 4 waves per workgroup (several workgroups per CU) unless a row needs more waves than that
    const int wpr = best.TS > 64 ? best.TS / 64 : 1;
    best.nwaves = wpr * (4 / wpr > 0 ? 4 / wpr : 1);
    return best;
}

// The tag-stream kernel multiplies up to 8 activation rows per pass (every codeword gathered once, one x gather
// per row).  With column orders (where the alternative is the VALU kernel) it is used for any B <= 32.  Without,
// it wins over the matrix-core kernel's single L2 gather per tag up to 4 rows on every shape, and up to 8 rows
// when a row's part of x is short enough for several rows per pass.  Measured on the 7B layer (microseconds,
// stream / matrix-core kernel): q|k|v 13.8 / 26.7 at 2 rows, 14.5 / 27.1 at 4, 18.6 / 26.8 at 8; o 12.5 / 15.0, 13.7 /
// 14.9, 17.6 / 15.4; gate|up 24.7 / (85 at any row count), 33.5, 62.8; down (rows of 2368 chunks) 18.3, 33.4 / (52 at
// any row count), 63.2.
static bool stream_rows(const sq_matrix& m, int B) {
    if (!stream_shape(m)) return false;
    if (!m.tags) return true;                                    // one-copy residency: the stream is all there is
    return B <= 4 || m.perms != nullptr || (B <= 8 && m.C / m.d <= 1024);
}

// ---- matrix-core path (pieces without column orders)
struct MmaPlan { int RW, NT, KW, ks; };

static bool mma_shape(const sq_matrix& m) { return fast_shape(m) && !m.perms; }

// bytes of codebook the matrix-core kernel stages in LDS (0: gathers go through the cache)
static size_t mma_table_bytes(const sq_matrix& m) {
    const size_t tab = (size_t)m.G * ((size_t)1 << m.bits) * m.d * 2;
    return tab <= 128 * 1024 ? tab : 0;
}

// Rounds per wave, waves per workgroup and workgroup-level column slices that cover ceil(U / 4) rounds
// with the fewest idle rounds (ties: more rounds per wave, i.e. fewer waves to add up).
static MmaPlan mma_plan(const sq_matrix& m, int B) {
    const int ud = unit_dwords(m.bits), tpu = ud * 32 / m.bits, spu = tpu / (8 / m.d);
    const int rounds = (m.W / ud + 3) / 4, r1 = 32 / spu;
    MmaPlan best{0, 0, 0, 0};
    double best_cost = 1e30;
    const int NT = B > 16 ? 2 : 1;
    // waves per workgroup: 8 (16 for the variants with few activation operands per lane, which fit four waves per SIMD),
    // or as many as leave room in the CU's 160 KB of LDS, next to a codebook that is staged there (4 books of 4096 d = 4
    // entries fill 128 KB), for their accumulators of the tiles in flight and their activation staging areas.  Long rows
    // then take more, shorter column slices: 7B down, 148 rounds, at 4 rows: 15.1 us with 15 waves x 2 rounds x 5 slices
    // against 18.4 with 7 x 8 x 3, reduction launch included.
    const size_t tab = mma_table_bytes(m);
    for (int rw = NT == 1 ? r1 : r1 / 2; rw >= 1 && rw >= r1 / 4; rw /= 2) {
        const int need = (rounds + rw - 1) / rw;
        int mk = 8;
        if (tab) {
            const size_t room = 160 * 1024 - tab - 16;
            const size_t per_wave = std::max((size_t)64 * NT * 16 * mma_pft(rw), (size_t)mma_x_stage_bytes(tpu * m.d));
            mk = (int)std::min<size_t>(mma_waves_max(rw * spu * NT, true), room / per_wave);
            if (mk < 1) continue;
        }
        const int ks = (need + mk - 1) / mk, kw = (need + ks - 1) / ks;
        const double cost = (double)rw * kw * ks / rounds + 0.03 * (ks - 1) + 0.002 * kw;
        if (cost < best_cost - 1e-9) { best_cost = cost; best = MmaPlan{rw, NT, kw, ks}; }
    }
    return best;
}

// Passes of 32 rows through the matrix-core decode kernel against decode + tile GEMM (7B layer): 77 us per pass
// against 600-640 us when the codebook sits in LDS (d = 4), 201 us per pass when its gathers go to L2.  A
// codebook that fills most of LDS leaves room for fewer waves per workgroup and doubles the cost of a pass
// (27B layer, 4 books of 4096: 246 us per pass against 800 us).
int small_pass_limit(const sq_matrix* mats, int n) {
    int limit = 224;
    for (int i = 0; i < n; ++i) {
        if (!mma_shape(mats[i])) return 0;
        const size_t tab = mma_table_bytes(mats[i]);
        const int li = tab == 0 ? 64 : tab > 64 * 1024 ? 96 : 224;
        if (li < limit) limit = li;
    }
    return n > 0 ? limit : 0;
}

static size_t mma_part_bytes(const sq_matrix& m, int B) {
    const MmaPlan pl = mma_plan(m, B);
    return pl.ks > 1 ? ((((size_t)pl.ks * B * m.R * 4) + 255) & ~(size_t)255) : 0;
}

size_t small_workspace(const sq_matrix* mats, int n, int B) {
    size_t tot = 0;
    for (int i = 0; i < n; ++i) {
        if (stream_rows(mats[i], B)) continue;                   // its partial sums live in the workspace header
        if (mma_shape(mats[i])) tot += mma_part_bytes(mats[i], B);
        else if (mats[i].perms && fast_shape(mats[i])) tot += xp_bytes(mats[i], B);
    }
    return tot;
}

bool small_uses_sums(const sq_matrix* mats, int n) {
    for (int i = 0; i < n; ++i)
        if (mats[i].R > 0 && stream_shape(mats[i])) return true;
    return false;
}

// Pieces [0, cnt) share format and row length: one persistent launch (+ one reduction per piece if ks > 1).
static int launch_mma_group(const sq_matrix* mats, int cnt, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                            int64_t ldy, int B, char* ws, size_t& ws_off, int cus, hipStream_t s) {
    const sq_matrix& m0 = mats[0];
    const MmaPlan pl = mma_plan(m0, B);
    MmaArgs a;
    a.n = cnt;
    a.x = (const uint16_t*)x; a.ldx = ldx; a.y = y; a.ldy = ldy; a.B = B; a.x_dtype = x_dtype; a.y_dtype = y_dtype;
    a.U = m0.W / unit_dwords(m0.bits);
    a.ks = pl.ks;
    a.table_bytes = (int)mma_table_bytes(m0);
    const int threads = pl.KW * 64;
    // LDS behind the codebook: the waves' accumulators of the tiles between two barriers (MMA_TT tiles when the codebook
    // is read through the cache; with the codebook in LDS as many as the workgroup walks, if they fit: sized below)
    const size_t red_tile = (size_t)pl.KW * 64 * pl.NT * 16;
    const int pft = mma_pft(pl.RW);
    a.tg = a.table_bytes ? pft : 0;
    const int tpu = unit_dwords(m0.bits) * 32 / m0.bits;
    const size_t xstage = (size_t)pl.KW * mma_x_stage_bytes(tpu * m0.d);      // the waves' activation staging areas (same LDS)
    size_t smem = (size_t)a.table_bytes + 16 + std::max(xstage, a.table_bytes ? (size_t)a.tg * red_tile : pl.KW > 1 ? (size_t)MMA_TT * red_tile : 0);
    int rc = SQ_EUNSUPPORTED;
#define SQ_CASE(BI, DD) if (m0.bits == BI && m0.d == DD) rc = launch_mma_b##BI##d##DD(OP, a, pl.RW, pl.NT, GRID, threads, smem, s)
#define OP 1
#define GRID 0
    SQ_CASE(16, 8); SQ_CASE(12, 4); SQ_CASE(10, 4); SQ_CASE(8, 4);
#undef OP
#undef GRID
    if (rc < 1) return rc < 0 ? rc : fail(SQ_ELAUNCH, "sq_linear_small: kernel does not fit a CU");
    const int slots = cus * rc;                                  // workgroups resident at once
    int64_t rows_total = 0;
    for (int k = 0; k < cnt; ++k) rows_total += mats[k].R;
    int wg = 0;
    for (int k = 0; k < cnt; ++k) {
        MmaPiece& P = a.p[k];
        P.m = mats[k];
        const sq_matrix& mk = mats[k];
        P.tiled = mk.stream && !mk.perms && tiled_format_ok(mk.R, mk.W, mk.C, mk.d, mk.bits) && ((uintptr_t)mk.stream & 15) == 0
                      ? (const uint32_t*)mk.stream : nullptr;
        P.part = nullptr;
        if (pl.ks > 1) {
            P.part = (float*)(ws + ws_off);
            ws_off += mma_part_bytes(mats[k], B);
        }
        const int ntiles = (mats[k].R + 15) / 16;
        int nshare = (int)((mats[k].R * (int64_t)slots / rows_total) / pl.ks);
        if (nshare > ntiles) nshare = ntiles;
        if (nshare < 1) nshare = 1;
        P.wg_begin = wg;
        P.wg_count = nshare * pl.ks;
        wg += P.wg_count;
    }
    for (int k = cnt; k < GEMV_MAX_PIECES; ++k) a.p[k] = a.p[0];
    if (a.table_bytes) {
        int most = 1;                                            // most tiles one workgroup walks
        for (int k = 0; k < cnt; ++k) {
            const int ntiles = (mats[k].R + 15) / 16, nshare = a.p[k].wg_count / pl.ks;
            most = std::max(most, (ntiles + nshare - 1) / nshare);
        }
        const size_t room = (size_t)(160 * 1024) / rc - a.table_bytes - 16;
        int fit = (int)(room / red_tile) / pft * pft;
        a.tg = std::min((most + pft - 1) / pft * pft, std::max(fit, pft));
        smem = (size_t)a.table_bytes + 16 + std::max(xstage, (size_t)a.tg * red_tile);
    }
#define OP 0
#define GRID wg
    rc = SQ_EUNSUPPORTED;
    SQ_CASE(16, 8); SQ_CASE(12, 4); SQ_CASE(10, 4); SQ_CASE(8, 4);
#undef OP
#undef GRID
#undef SQ_CASE
    if (rc) return rc;
    if (pl.ks > 1)
        for (int k = 0; k < cnt; ++k) {
            const sq_matrix& mk = mats[k];
            hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((B * mk.R + 255) / 256)), dim3(256), 0, s,
                               a.p[k].part, pl.ks, B, mk.R, mk.row_scale, y, ldy, mk.y_off, y_dtype);
            rc = check_launch("sq_linear_small(splitk_reduce)");
            if (rc) return rc;
        }
    return SQ_OK;
}

// (Pieces with column orders would gather the producer's three operands through every order of a run from memory:
// measured 39.9 against 21.4 us for the stand-alone add + norm followed by the product on the masked 27B q|k|v stack,
// 43.5 against 30.6 us on gate|up.  They take the two launches.)
bool small_fuses_producer(const sq_matrix* mats, int n, int B) {
    if (B != 1 || n < 1 || n > GEMV_MAX_PIECES_STREAM) return false;
    for (int i = 0; i < n; ++i)
        if (mats[i].R <= 0 || !stream_rows(mats[i], 1) || mats[i].bits != mats[0].bits || mats[i].G != mats[0].G || mats[i].perms) return false;
    return true;
}

// SiLU(gate) * up written by the product itself: the two pieces are a gate and an up projection of one shape on the
// tag-stream kernel (no column orders, cut into the same runs), at most 8 activation rows (one pass)
bool small_fuses_silu(const sq_matrix* mats, int n, int B) {
    if (n != 2 || B < 1 || B > 8) return false;
    const sq_matrix &g = mats[0], &u = mats[1];
    if (g.R <= 0 || g.R != u.R || g.C != u.C || g.bits != u.bits || g.G != u.G || g.perms || u.perms) return false;
    // (the same cut into runs; the other fields of stream_runs describe each piece's own buffer and may differ)
    if (!stream_rows(g, B) || !stream_rows(u, B) || stream_runs_of(g) != stream_runs_of(u) || stream_run_max_of(g) != stream_run_max_of(u) ||
        g.stream_groups != u.stream_groups)
        return false;
    if (stream_geom_of(g).NV > 16 || stream_group_len(mats, 2) != 2) return false;
    return stream_pass_rows(B) >= B;
}

int launch_small_silu(const sq_matrix* mats, int n, const void* x, int x_dtype, int64_t ldx, void* act, int64_t ld_act, int B,
                      void* sums, hipStream_t s, const sq_producer* from) {
    const bool x_ok = (B == 1 || ldx % 8 == 0) && (((uintptr_t)x & 15) == 0);
    if (!small_fuses_silu(mats, n, B) || !(x_ok || from) || (from && !small_fuses_producer(mats, n, B)))
        return fail(SQ_EUNSUPPORTED, "sq_linear_small_silu: no fused kernel for this stack (run sq_linear_small, then sq_silu_mul)");
    if (!sums) return fail(SQ_EWORKSPACE, "sq_linear_small_silu: these pieces need a workspace (its header holds their partial sums)");
    return launch_stream_group(mats, 2, x, x_dtype, ldx, nullptr, x_dtype, 0, B, (char*)sums, s, from, act, ld_act);
}

int launch_small(const sq_matrix* mats, int n, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                 int64_t ldy, int B, void* ws, size_t ws_bytes, void* sums, hipStream_t s, const sq_producer* from) {
    if (from && !small_fuses_producer(mats, n, B)) return fail(SQ_EUNSUPPORTED, "sq_linear_small_from: no fused kernel for this stack");
    if (small_workspace(mats, n, B) > ws_bytes)
        return fail(SQ_EWORKSPACE, "sq_linear_small: workspace %zu < %zu", ws_bytes, small_workspace(mats, n, B));
    const int cus = device_cus();
    const bool x_ok = (B == 1 || ldx % 8 == 0) && (((uintptr_t)x & 15) == 0);   // 16-byte activation loads
    size_t ws_off = 0;
    int i = 0;
    while (i < n) {
        const sq_matrix& m0 = mats[i];
        if (m0.R == 0) { ++i; continue; }
        const int ud = unit_dwords(m0.bits);
        if (stream_rows(m0, B) && (x_ok || from)) {
            if (!sums) return fail(SQ_EWORKSPACE, "sq_linear_small: these pieces need a workspace (its header holds their partial sums)");
            int j = i + 1;
            while (j < n && j - i < GEMV_MAX_PIECES_STREAM && stream_rows(mats[j], B) && mats[j].bits == m0.bits && mats[j].G == m0.G && mats[j].R > 0) ++j;
            j = i + stream_group_len(mats + i, j - i);
            int rc = launch_stream_group(mats + i, j - i, x, x_dtype, ldx, y, y_dtype, ldy, B, (char*)sums, s, from);
            if (rc) return rc;
            i = j;
            continue;
        }
        if (B <= 2 && x_ok && segs_shape(m0) && (B == 1 || mma_table_bytes(m0) > 64 * 1024)) {
            // d = 4 rows of whole segments at one activation row, and at two when the codebooks leave a CU room for one
            // workgroup only: the row-segment kernel (7B-shaped layer, 12-bit tags: 41.7 us at one row against 50 on the
            // matrix-core kernel, 52.4 against 49.8 at two; four codebooks of 4096: 71-73 against 78-83 at two)
            int j = i + 1;
            while (j < n && j - i < 4 && segs_shape(mats[j]) && mats[j].W == m0.W && mats[j].G == m0.G) ++j;
            if (segs_fits(mats + i, j - i, B, cus)) {
                int rc = launch_segs_group(mats + i, j - i, x, x_dtype, ldx, y, y_dtype, ldy, B, cus, s);
                if (rc) return rc;
                for (int k = i; k < j; ++k) ws_off += mma_part_bytes(mats[k], B);   // (what small_workspace counted for them)
                i = j;
                continue;
            }
        }
        if (mma_shape(m0) && x_ok) {
            int j = i + 1;
            while (j < n && j - i < GEMV_MAX_PIECES && mma_shape(mats[j]) && mats[j].bits == m0.bits && mats[j].d == m0.d &&
                   mats[j].W == m0.W && mats[j].G == m0.G && mats[j].R > 0)
                ++j;
            int rc = launch_mma_group(mats + i, j - i, x, x_dtype, ldx, y, y_dtype, ldy, B, (char*)ws, ws_off, cus, s);
            if (rc) return rc;
            i = j;
            continue;
        }
        const Plan pl = (fast_shape(m0) && x_ok) ? plan_for(m0.W / ud, m0.bits, m0.d) : Plan{0, 0, 0};
        if (pl.TS == 0 && !m0.tags)
            return fail(SQ_EUNSUPPORTED, "sq_linear_small: a matrix held as its tag stream only needs 16-byte aligned x with ldx %% 8 == 0");
        if (pl.TS == 0) {
            int rc = launch_small_generic(mats + i, 1, x, x_dtype, ldx, y, y_dtype, ldy, B, s);
            if (rc) return rc;
            if (stream_rows(m0, B)) {}
            else if (mma_shape(m0)) ws_off += mma_part_bytes(m0, B);
            else if (m0.perms && fast_shape(m0)) ws_off += xp_bytes(m0, B);
            ++i;
            continue;
        }
        // pieces i .. j-1 share one launch when their format, geometry and codebook size agree
        const int U = m0.W / ud;
        const size_t tab0 = (size_t)m0.G * ((size_t)1 << m0.bits) * m0.d * 2;
        int j = i + 1;
        while (j < n && j - i < GEMV_MAX_PIECES && fast_shape(mats[j]) && mats[j].bits == m0.bits && mats[j].d == m0.d &&
               mats[j].W == m0.W && mats[j].G == m0.G && mats[j].R > 0)
            ++j;
        GemvArgs a;
        a.n = j - i;
        a.x = (const uint16_t*)x; a.ldx = ldx; a.y = y; a.ldy = ldy; a.B = B;
        a.x_dtype = x_dtype; a.y_dtype = y_dtype; a.TS = pl.TS;
        a.table_bytes = tab0 <= 128 * 1024 ? (int)tab0 : 0;
        const int wpr = pl.TS > 64 ? pl.TS / 64 : 1;
        int64_t rows_total = 0;
        for (int k = i; k < j; ++k) rows_total += mats[k].R;
        for (int k = i; k < j; ++k) {
            GemvPiece& P = a.p[k - i];
            P.m = mats[k];
            P.U = U;
            P.xp = nullptr;
            if (mats[k].perms) {
                uint16_t* xp = (uint16_t*)((char*)ws + ws_off);
                ws_off += xp_bytes(mats[k], B);
                const int Mx = mats[k].M > 1 ? mats[k].M : 1;
                const int64_t tot = (int64_t)Mx * B * mats[k].C;
                hipLaunchKernelGGL(permute_x_kernel, dim3((unsigned)((tot + 255) / 256)), dim3(256), 0, s,
                                   (const uint16_t*)x, ldx, x_dtype, mats[k].perms, Mx, B, mats[k].C, xp);
                int rc = check_launch("sq_linear_small(permute_x)");
                if (rc) return rc;
                P.xp = xp;
            }
        }
        for (int k = j - i; k < GEMV_MAX_PIECES; ++k) a.p[k] = a.p[0];
        for (int b0 = 0; b0 < B;) {
            const int left = B - b0;
            int nbt = left >= 4 ? 4 : left >= 2 ? 2 : 1;
            // fewer activation rows per pass when the registers or the workgroup width do not allow more
            while (nbt > 1 && (cfg_xw(m0.bits, m0.d, pl.S, nbt) > 192 || cfg_lb(m0.bits, m0.d, pl.S, nbt) < wpr * 64)) nbt >>= 1;
            const int lb = cfg_lb(m0.bits, m0.d, pl.S, nbt);
            int nwaves = pl.nwaves;
            // a codebook that leaves room for one workgroup per CU: make that workgroup as wide as allowed
            if (nwaves * 64 > lb || a.table_bytes > 80 * 1024) nwaves = (lb / 64) / wpr * wpr;
            const int ngrp = pl.TS > 64 ? nwaves / wpr : nwaves * (64 / pl.TS);
            const size_t smem = (size_t)a.table_bytes + (wpr > 1 ? (size_t)GEMV_PF * ngrp * wpr * nbt * sizeof(float) : 0);
            // persistent grid: workgroups per CU bounded by LDS and wave slots, split over the pieces by rows
            int rc = SQ_EUNSUPPORTED;
#define SQ_CASE(BI, DD) if (m0.bits == BI && m0.d == DD) rc = launch_gemv_b##BI##d##DD(OP, a, pl.S, nbt, GRID, nwaves * 64, smem, s)
#define OP 1
#define GRID 0
            SQ_CASE(16, 8); SQ_CASE(12, 4); SQ_CASE(10, 4); SQ_CASE(8, 4);      // workgroups that fit on a CU
#undef OP
#undef GRID
            if (rc < 1) return rc < 0 ? rc : fail(SQ_ELAUNCH, "sq_linear_small: kernel does not fit a CU");
            const int per_cu = rc;
            const int64_t row_quant = (int64_t)ngrp * GEMV_PF;
            const int grid_target = cus * per_cu;
            int wg_begin = 0;
            for (int k = i; k < j; ++k) {
                GemvPiece& P = a.p[k - i];
                int cnt = (int)((mats[k].R * (int64_t)grid_target + rows_total - 1) / rows_total);
                const int most = (int)((mats[k].R + row_quant - 1) / row_quant);
                if (cnt > most) cnt = most;
                if (cnt < 1) cnt = 1;
                P.wg_begin = wg_begin;
                P.wg_count = cnt;
                wg_begin += cnt;
            }
            a.b0 = b0;
            rc = SQ_EUNSUPPORTED;
#define OP 0
#define GRID wg_begin
            SQ_CASE(16, 8); SQ_CASE(12, 4); SQ_CASE(10, 4); SQ_CASE(8, 4);
#undef OP
#undef GRID
#undef SQ_CASE
            if (rc) return rc;
            b0 += nbt;
        }
        i = j;
    }
    return SQ_OK;
}

}  // namespace sq
