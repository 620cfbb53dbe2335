// Bucketed tag stream: the batch-1 product for codebooks too large for LDS (K = 8192 .. 65,536 at d = 8; several
// codebooks per matrix count as one long codebook, see sq_stream.h).
//
// A 65,536 x 8 fp16 codebook is 1 MiB; gathering 16-byte codewords from it through L2 is what bounds the
// row-major kernels.  Here the tags of a matrix are regrouped once, at load time, by the part of the
// codebook they point into, so that every workgroup gathers from a 64 KB slice held in LDS:
//
//   bucket (kp, s)   column part kp (PC chunks of d columns each) x codebook slice s (tags s*4096 .. +4095)
//   entry            tag & 4095 | (chunk - kp * PC) << 12: 24 bits, or 21 when the part has at most 496 chunks
//   lane task        the entries of one row in one bucket (about C/d / (KP * NS) of them)
//
// Rows are first ordered by column order (row_mask, stable), so that consecutive rows share one; each column
// order's rows are cut into groups of 64 (the last group of an order may be short) and into runs of at most GR
// groups, one workgroup per (bucket, run); the caller picks the number of runs so that the pieces it launches
// together make about one workgroup (of 16 waves) per CU.  Within a bucket the rows of a run are sorted by entry count
// (descending, stable): one lane per row, one wave per group.  A group is stored as steps of 64 x 12 bytes
// (4 entries of 24 bits per lane and step, lane-major, so a wave reads 768 contiguous bytes per step) or of 64 x 8
// bytes (3 entries of 21 bits), padded to the longest row of the group; sorting keeps that padding at 5 to 7 percent
// of a large matrix.  A workgroup stages its slice and its part of x
// (gathered through the run's column order, if any) in LDS; each lane accumulates dot(codeword, x chunk) over
// its entries in fp32 and leaves one partial sum per (bucket, row) in the workspace header, whose words are zero
// between launches: a partial sum is its own arrival flag.  The workgroups of all buckets that cover the same run
// each take a share of the run's rows, read the NS * KP partials of a row until none is zero, add them in a fixed
// order (so results do not depend on scheduling), apply the row scale, store y and put zero back.
//
// Stream buffer (one allocation; offsets follow from C/d, the tag width, the group and run counts):
//   heads  uint32 [NV * NG][4]    {rest, nst, unit0, split | g0 << 8} of every group (NV = KP * NS buckets, NG groups per
//                                 bucket, bucket v = kp * NS + s): where its steps are, see sq_stream.h
//   slots  uint16 [NV * NG * 64]  the lane's place counted from its run's first place (place = the row's index in `rows`
//                                 below; 0x1FFF: a lane without a row) | 0x2000 when the row has entries in the bucket;
//                                 lanes 64 g .. 64 g + 63 of a bucket are group g
//   runs   [runs] x 32 bytes       first group, group count, column orders of the run, index of its first unit; first
//                                 group (within the run) and id of each of up to 8 column orders (one byte each)
//   rows   uint32 [NG * 64]       the rows ordered by column order, 64 per group (0x7FFFF where a group is short):
//                                 places 64 g0 .. 64 (g0 + ng) - 1 are a run's rows, and partial sums are indexed by place
//   steps  [total][64][12 | 8]    entries: the first-steps region (FS steps per unit and bucket), then the rest
#include <algorithm>
#include <atomic>
#include <mutex>
#include <string.h>
#include <thread>
#include <vector>
#include "sq_stream.h"

constexpr int STREAM_CLIMB = 1;      // hill-climbing passes of the entry ordering (load time against LDS collisions)

namespace sq {

// A run: groups g0 .. g0 + ng - 1 of every bucket.  Its rows belong to `norders` column orders (one without row orders);
// the groups of order[i] begin at group bound[i] of the run (bound[0] = 0), and the kernel keeps copy i of x, gathered
// through that order, in LDS for them.
// u0: the index of the run's first unit (units are counted run after run).
struct StreamRun { int32_t g0, ng, norders, u0; uint8_t bound[STREAM_RUN_ORDERS]; uint8_t order[STREAM_RUN_ORDERS]; };
static_assert(sizeof(StreamRun) == 32, "run records are read as 8 dwords");

StreamGeom stream_geom(int C, int d, int bits, int groups, int runs, bool balanced, int fs) {
    StreamGeom g;
    g.U = C / d;
    g.NS = 1 << (bits - STREAM_SLICE_BITS);
    g.KP = (g.U + STREAM_PART_MAX - 1) / STREAM_PART_MAX;
    g.PC = (g.U + g.KP - 1) / g.KP;
    g.NV = g.NS * g.KP;
    g.NG = groups;
    g.runs = runs;
    g.fmt = stream_fmt(g.PC);
    g.fs = fs < 1 ? g.fmt.pf : fs < g.fmt.pf ? fs : g.fmt.pf;
    g.off_slots = ((size_t)g.NV * g.NG * 16 + 255) & ~(size_t)255;          // four words per (bucket, group)
    g.off_runs = (g.off_slots + (size_t)g.NV * g.NG * 64 * 2 + 255) & ~(size_t)255;
    g.off_rows = (g.off_runs + (size_t)runs * sizeof(StreamRun) + 255) & ~(size_t)255;
    size_t end = (g.off_rows + (size_t)g.NG * 64 * 4 + 255) & ~(size_t)255;
    g.off_table = g.off_unmap = 0;
    if (balanced) {
        g.off_table = end;
        g.off_unmap = end + ((size_t)d * 2 << bits);
        end = (g.off_unmap + ((size_t)2 << bits) + 255) & ~(size_t)255;
    }
    g.off_steps = end;
    g.total_steps = 0;
    return g;
}

// (R + 64 * 256 bounds the places: every column order can leave one group short)
bool stream_format_ok(int R, int C, int d, int bits, int G) {
    if (G < 1 || (G & (G - 1)) != 0 || bits < 1 || bits > 16) return false;
    const int lb = stream_label_bits(bits, G);
    return d == 8 && lb > STREAM_SLICE_BITS && (1 << (lb - STREAM_SLICE_BITS)) <= (G > 1 ? STREAM_SLICES_MAX : 16) && C % d == 0 &&
           R > 0 && R + 64 * 256 < (int)STREAM_NO_ROW;
}

static inline uint32_t host_tag(const uint32_t* row, int W, int bits, int j) {
    const int64_t p = (int64_t)j * bits;
    const int w = (int)(p >> 5), s = (int)(p & 31);
    uint64_t v = row[w];
    if (s + bits > 32 && w + 1 < W) v |= (uint64_t)row[w + 1] << 32;
    return (uint32_t)(v >> s) & ((1u << bits) - 1u);
}

static void parallel_rows(int R, const std::function<void(int, int)>& fn) {
    unsigned nt = std::thread::hardware_concurrency();
    if (nt < 1) nt = 1;
    if (nt > 16) nt = 16;
    if ((unsigned)R < nt * 64) nt = 1;
    if (nt == 1) { fn(0, R); return; }
    std::vector<std::thread> th;
    const int per = (R + (int)nt - 1) / (int)nt;
    for (unsigned t = 0; t < nt; ++t) {
        const int a = (int)t * per, b = std::min(R, a + per);
        if (a < b) th.emplace_back(fn, a, b);
    }
    for (auto& t : th) t.join();
}


struct StreamPlan {
    StreamGeom g;
    int GR;                          // groups in the longest run
    int orders_max;                  // most column orders in one run
    std::vector<StreamRun> runs;
    std::vector<uint32_t> base;      // [NG * 64]: rows ordered by column order, STREAM_NO_ROW where a group is short
    std::vector<uint16_t> cnt;       // [NV][R]
    std::vector<uint32_t> pos;       // [NV][R]: lane position (group * 64 + lane) of row r in bucket v
    std::vector<uint32_t> goff;      // [NV * NG + 1]: the groups' steps counted bucket after bucket, group after group (how the
                                     // builder lays them out before they move to their places)
    uint64_t logical_steps;          // goff[NV * NG]
    int NU;                          // units of one bucket
    std::vector<uint32_t> slot32;    // [NV * NG * 64]: place | count << STREAM_ROW_BITS per lane (STREAM_NO_ROW: no row), the
                                     // builder's own form of the slots
    std::vector<uint32_t> run_of;    // [NG]: the run of a group
    std::vector<uint32_t> head4;     // [NV * NG][4]: {rest, nst, unit0, split}, what the buffer holds per (bucket, group)
    std::vector<uint16_t> remap;     // balanced streams: file id -> new id (empty: identity)
};

// Relabelling of the codewords for a stream with a codebook of its own: the codewords are dealt, most used first, to
// whichever slice of 4096 carries the fewest tags so far and still has room, so every slice ends up with the same
// share of the tags (a slice is one workgroup's work) whatever the distribution of the tags is, and a slice's popular
// codewords get consecutive places, i.e. different LDS bank groups.
// With several codebooks (row_book names a row's) every codebook is relabelled by itself, over its own slices:
// remap[book << bits | label] is the new label within the book; a codebook of at most one slice keeps its labels.
static void balance_codewords(const uint32_t* tags, int R, int W, int U, int bits, std::vector<uint16_t>& remap, int G = 1,
                              const uint8_t* row_book = nullptr) {
    const int K = 1 << bits, NS = K >> STREAM_SLICE_BITS, SL = 1 << STREAM_SLICE_BITS;
    remap.assign((size_t)G * K, 0);
    if (NS < 2) {
        for (size_t k = 0; k < remap.size(); ++k) remap[k] = (uint16_t)(k & (size_t)(K - 1));
        return;
    }
    std::vector<uint64_t> count((size_t)G * K, 0);
    for (int r = 0; r < R; ++r) {
        const uint32_t* row = tags + (size_t)r * W;
        uint64_t* cb = count.data() + (size_t)(row_book ? row_book[r] & (G - 1) : 0) * K;
        for (int j = 0; j < U; ++j) ++cb[host_tag(row, W, bits, j)];
    }
    std::vector<uint32_t> ids(K);
    std::vector<uint64_t> load(NS);
    std::vector<int> fill(NS);
    for (int b = 0; b < G; ++b) {
        const uint64_t* cb = count.data() + (size_t)b * K;
        for (int k = 0; k < K; ++k) ids[k] = (uint32_t)k;
        std::stable_sort(ids.begin(), ids.end(), [cb](uint32_t x, uint32_t y) { return cb[x] > cb[y]; });
        std::fill(load.begin(), load.end(), 0);
        std::fill(fill.begin(), fill.end(), 0);
        for (int k = 0; k < K; ++k) {
            int best = -1;
            for (int sl = 0; sl < NS; ++sl)
                if (fill[sl] < SL && (best < 0 || load[sl] < load[best])) best = sl;
            remap[(size_t)b * K + ids[k]] = (uint16_t)(best * SL + fill[best]);
            ++fill[best];
            load[best] += cb[ids[k]];
        }
    }
}

// (G > 1: the labels a row's tags become are book << bits | tag, see sq_stream.h; `balanced` is for one codebook only)
static void plan_stream(const uint32_t* tags, int R, int W, int C, int d, int bits, const uint8_t* row_mask, int runs,
                        StreamPlan& P, bool balanced, int G, const uint8_t* row_book) {
    const int lbits = stream_label_bits(bits, G);
    P.remap.clear();
    if (balanced) balance_codewords(tags, R, W, C / d, bits, P.remap);
    const uint16_t* remap = balanced ? P.remap.data() : nullptr;
    // rows by column order, groups and runs
    std::vector<uint32_t> order(R);
    for (int r = 0; r < R; ++r) order[r] = (uint32_t)r;
    if (row_mask)
        std::stable_sort(order.begin(), order.end(), [row_mask](uint32_t a, uint32_t b) { return row_mask[a] < row_mask[b]; });
    StreamGeom g0 = stream_geom(C, d, lbits, 0, 0);
    if (runs <= 0) runs = (STREAM_DEFAULT_WGS + g0.NV / 2) / g0.NV;
    if (runs < 1) runs = 1;
    // Groups per column order.  A run takes the groups of one order, GR at a time, or, when orders are small, the whole
    // groups of up to `cap` orders that follow each other (a masked k projection has 64 rows per order: one run per order
    // would be 16 workgroups of one group each per bucket).  cap: as many gathered copies of x as fit LDS beside the slice
    // and the run's partial sums, and as the staging loop covers with four chunks per thread.
    std::vector<int> first, ngm;
    for (int a = 0; a < R;) {
        int b = a;
        const int m = row_mask ? row_mask[order[a]] : 0;
        while (b < R && (row_mask ? row_mask[order[b]] : 0) == m) ++b;
        first.push_back(a);
        ngm.push_back((b - a + 63) / 64);
        a = b;
    }
    first.push_back(R);
    int total_groups = 0;
    for (int q : ngm) total_groups += q;
    const int xs_bytes = g0.fmt.narrow ? 8192 : (g0.PC + 16) * 16;     // (stream_xs)
    int cap = (160 * 1024 - 65536 - STREAM_RUN_MAX * 256 - 1024) / xs_bytes;
    cap = std::min(cap, std::min(4, 4096 / g0.PC));            // (4: two activation rows per pass still fit LDS at C = 5120)
    if (cap < 1 || !row_mask) cap = 1;
    // the runs for a run length GR (into `out` if given): returns their number
    auto pack = [&](int GR, std::vector<StreamRun>* out, int* longest) {
        int64_t n = 0;
        StreamRun cur{0, 0, 0, 0, {0}, {0}};
        int gbase = 0, lg = 1;
        auto flush = [&]() {
            if (cur.ng > 0) { ++n; lg = std::max(lg, cur.ng); if (out) out->push_back(cur); }
            cur = StreamRun{0, 0, 0, 0, {0}, {0}};
        };
        for (size_t i = 0; i < ngm.size(); ++i) {
            const int q = ngm[i], m = row_mask ? row_mask[order[first[i]]] : 0;
            if (q > GR) {                                        // an order longer than a run: runs of its own
                flush();
                for (int p0 = 0; p0 < q; p0 += GR) {
                    cur = StreamRun{gbase + p0, std::min(GR, q - p0), 1, 0, {0}, {(uint8_t)m}};
                    flush();
                }
            } else if (cur.ng > 0 && cur.ng + q <= GR && cur.norders < cap) {
                cur.bound[cur.norders] = (uint8_t)cur.ng;
                cur.order[cur.norders] = (uint8_t)m;
                ++cur.norders;
                cur.ng += q;
            } else {
                flush();
                cur = StreamRun{gbase, q, 1, 0, {0}, {(uint8_t)m}};
            }
            gbase += q;
        }
        flush();
        if (longest) *longest = lg;
        return n;
    };
    // GR = the fewest groups per run that keep the run count within the request.  A run's partial sums are staged in
    // LDS: no run longer than STREAM_RUN_MAX groups (more runs than asked for then).
    int GR = 1;
    while (GR < STREAM_RUN_MAX && GR < total_groups && pack(GR, nullptr, nullptr) > runs) ++GR;
    // With one column order the kernel derives the cut from the run count alone, as ceil(groups / runs) per run: settle
    // on a run length that this formula gives back.
    if (ngm.size() == 1)
        for (;;) {
            const int n = (ngm[0] + GR - 1) / GR, g2 = (ngm[0] + n - 1) / n;
            if (g2 == GR) break;
            GR = g2;
        }
    P.runs.clear();
    P.base.clear();
    pack(GR, &P.runs, &P.GR);
    P.orders_max = 1;
    for (const StreamRun& run : P.runs) P.orders_max = std::max(P.orders_max, (int)run.norders);
    for (size_t i = 0; i < ngm.size(); ++i) {
        const int a = first[i], b = first[i + 1];
        for (int k = 0; k < ngm[i] * 64; ++k) P.base.push_back(a + k < b ? order[a + k] : STREAM_NO_ROW);
    }
    P.g = stream_geom(C, d, lbits, (int)(P.base.size() / 64), (int)P.runs.size(), balanced);
    const StreamGeom& g = P.g;
    P.cnt.assign((size_t)g.NV * R, 0);
    P.pos.assign((size_t)g.NV * R, 0);
    P.goff.assign((size_t)g.NV * g.NG + 1, 0);
    parallel_rows(R, [&](int a, int b) {
        for (int r = a; r < b; ++r) {
            const uint32_t* row = tags + (size_t)r * W;
            const uint32_t book = row_book ? (uint32_t)(row_book[r] & (G - 1)) << bits : 0u;
            for (int j = 0; j < g.U; ++j) {
                uint32_t t = host_tag(row, W, bits, j);
                if (remap) t = remap[t];
                t |= book;
                const int v = (j / g.PC) * g.NS + (int)(t >> STREAM_SLICE_BITS);
                ++P.cnt[(size_t)v * R + r];
            }
        }
    });
    std::vector<uint32_t> steps((size_t)g.NV * g.NG, 0);
    parallel_rows(g.NV, [&](int a, int b) {
        std::vector<uint32_t> rows;
        for (int v = a; v < b; ++v) {
            const uint16_t* c = &P.cnt[(size_t)v * R];
            for (const StreamRun& run : P.runs) {
                // rows move between the groups of one column order only: a group reads one copy of x
                for (int oi = 0; oi < run.norders; ++oi) {
                    const int ga = run.g0 + run.bound[oi], gb = run.g0 + (oi + 1 < run.norders ? run.bound[oi + 1] : run.ng);
                    rows.clear();
                    for (int k = ga * 64; k < gb * 64; ++k)
                        if (P.base[k] != STREAM_NO_ROW) rows.push_back(P.base[k]);
                    std::stable_sort(rows.begin(), rows.end(), [c](uint32_t x, uint32_t y) { return c[x] > c[y]; });
                    for (size_t k = 0; k < rows.size(); ++k) P.pos[(size_t)v * R + rows[k]] = (uint32_t)(ga * 64 + k);
                    for (size_t k = 0; k < rows.size(); k += 64)
                        steps[(size_t)v * g.NG + ga + k / 64] = (c[rows[k]] + (uint32_t)g.fmt.eps - 1u) / (uint32_t)g.fmt.eps;
                }
            }
        }
    });
    uint64_t tot = 0;
    for (size_t k = 0; k < steps.size(); ++k) { P.goff[k] = (uint32_t)tot; tot += steps[k]; }
    P.goff[steps.size()] = (uint32_t)tot;
    P.logical_steps = tot;
    // Units and places: the first-steps region (NU units x NV buckets x FS steps) comes first, the groups'
    // remaining steps follow bucket after bucket, group after group.
    P.NU = 0;
    P.run_of.assign(g.NG, 0);
    for (size_t ri = 0; ri < P.runs.size(); ++ri) {
        StreamRun& run = P.runs[ri];
        run.u0 = P.NU;
        P.NU += run.ng * stream_split_of(run.ng);
        for (int k = 0; k < run.ng; ++k) P.run_of[run.g0 + k] = (uint32_t)ri;
    }
    // FS: the longest unit's step count, at most the prefetch depth
    const uint32_t PF = (uint32_t)g.fmt.pf;
    uint32_t fs = 1;
    for (int v = 0; v < g.NV; ++v)
        for (int gi = 0; gi < g.NG; ++gi) {
            const uint32_t split = (uint32_t)stream_split_of(P.runs[P.run_of[gi]].ng), nst = steps[(size_t)v * g.NG + gi];
            fs = std::max(fs, std::min(PF, (nst + split - 1) / split));
        }
    P.g.fs = (int)fs;
    P.head4.assign((size_t)g.NV * g.NG * 4, 0);
    uint64_t at = (uint64_t)P.NU * g.NV * fs;
    for (int v = 0; v < g.NV; ++v)
        for (int gi = 0; gi < g.NG; ++gi) {
            const StreamRun& run = P.runs[P.run_of[gi]];
            const uint32_t split = (uint32_t)stream_split_of(run.ng), nst = steps[(size_t)v * g.NG + gi];
            uint32_t* h = &P.head4[((size_t)v * g.NG + gi) * 4];
            h[0] = (uint32_t)at;
            h[1] = nst;
            h[2] = (uint32_t)run.u0 + (uint32_t)(gi - run.g0) * split;
            h[3] = split | ((uint32_t)run.g0 << 8);
            if (nst / split >= PF) at += nst - split * PF;
        }
    P.g.total_steps = at;
}

void stream_balance_host(const uint32_t* tags, int R, int W, int C, int d, int bits, uint16_t* remap_out, int G,
                         const uint8_t* row_book) {
    std::vector<uint16_t> remap;
    balance_codewords(tags, R, W, C / d, bits, remap, G, row_book);
    memcpy(remap_out, remap.data(), remap.size() * sizeof(uint16_t));
}

size_t stream_bytes_host(const uint32_t* tags, int R, int W, int C, int d, int bits, const uint8_t* row_mask, int runs,
                         const uint16_t* table, int G, const uint8_t* row_book) {
    StreamPlan P;
    plan_stream(tags, R, W, C, d, bits, row_mask, runs, P, table != nullptr, G, row_book);
    return P.g.off_steps + (size_t)P.g.total_steps * P.g.fmt.step_bytes;
}

// The lanes of a wave that one clock of a 16-byte LDS read serves.  A ds_read_b128 takes four clocks; measured on
// gfx950 (two lanes reading different rows of one bank group while every other lane reads a third address: one extra
// clock exactly for the pairs listed together here; 256 random address patterns then fit "sum over the four sets of
// the most distinct addresses in one group of four banks" to within 1 percent), the sets are not 16 consecutive lanes:
static const int LDS_CLOCK_LANES[4][16] = {
    {0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27},
    {4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31},
    {32, 33, 34, 35, 44, 45, 46, 47, 52, 53, 54, 55, 56, 57, 58, 59},
    {36, 37, 38, 39, 40, 41, 42, 43, 48, 49, 50, 51, 60, 61, 62, 63}};

// Orders the entries of the 16 lanes of one LDS clock (see the second pass of stream_build_host): every entry slot
// should hold, over the 16 lanes, 16 different codeword bank groups (tag mod 16) and 16 different bank groups of x
// (chunk mod 16).  A greedy fill (each lane takes the entry that collides least with the lanes before it) followed by
// hill climbing over the whole group: a lane that collides in a slot swaps that entry with one of its other slots when
// the two slots together get cheaper.
struct BankMatch {
    static constexpr uint32_t NONE = 0xFFFFFFFFu;
    std::vector<uint32_t> ent[16];           // [lane][slot]: the lane's real entries in slot order
    std::vector<uint8_t> ha, hb;             // [slot][16]: lanes per codeword / x bank group
    std::vector<uint8_t> mx;                 // [slot][4]: fullest codeword group, groups that full; the same for x
    uint32_t cnt[16];
    uint32_t eps = 4;                        // entries per lane and step (StreamFmt.eps)

    // entry n of a lane in a group whose steps begin at base: entries are kept one per word, [step][lane][eps], until
    // they are moved to their places
    uint32_t* rec_of(uint32_t* base, int lane, uint32_t n) const { return base + ((size_t)(n / eps) * 64 + lane) * eps + n % eps; }
    static int ga(uint32_t e) { return (int)(e & 15u); }
    static int gb(uint32_t e) { return (int)((e >> STREAM_SLICE_BITS) & 15u); }
    void add(uint32_t n, uint32_t e, int d) { ha[n * 16 + ga(e)] += d; hb[n * 16 + gb(e)] += d; }

    // zero_chunk: the first of the 16 chunks of x that the kernel keeps at zero
    void order_lanes(uint32_t* base, const uint32_t* sl, const int* lanes, uint32_t ns, uint32_t zero_chunk) {
        uint32_t most = 0;
        for (int l = 0; l < 16; ++l) {
            const uint32_t s0 = sl[lanes[l]];
            cnt[l] = (s0 & STREAM_NO_ROW) == STREAM_NO_ROW ? 0u : s0 >> STREAM_ROW_BITS;
            ent[l].resize(cnt[l]);
            for (uint32_t n = 0; n < cnt[l]; ++n) ent[l][n] = *rec_of(base, lanes[l], n);
            most = std::max(most, cnt[l]);
        }
        if (most == 0) return;
        ha.assign((size_t)ns * 16, 0);
        hb.assign((size_t)ns * 16, 0);
        // greedy fill, slot by slot; the lanes with the fewest entries left choose first
        int order[16];
        for (int l = 0; l < 16; ++l) order[l] = l;
        std::sort(order, order + 16, [this](int x, int y) { return cnt[x] != cnt[y] ? cnt[x] < cnt[y] : x < y; });
        for (uint32_t n = 0; n < most; ++n)
            for (int d = 0; d < 16; ++d) {
                const int l = order[d];
                if (cnt[l] <= n) continue;
                uint32_t bi = n;
                int bc = 1 << 30;
                for (uint32_t i = n; i < cnt[l]; ++i) {
                    const int c = ha[n * 16 + ga(ent[l][i])] + hb[n * 16 + gb(ent[l][i])];
                    if (c < bc) { bc = c; bi = i; if (c == 0) break; }
                }
                std::swap(ent[l][n], ent[l][bi]);
                add(n, ent[l][n], 1);
            }
        // Hill climbing.  What a slot costs is the fullest bank group of its codeword reads plus that of its x reads
        // (clocks); with 16 lanes on 16 bank groups some collisions are forced, and they are cheapest when they share
        // slots.  A lane in a fullest group swaps that entry with one of its other slots when the clocks of the two
        // slots together go down (ties: when the sum of squared group counts does).  The fullest group's count after
        // moving one lane from group p to group q follows from the count, the current maximum and how many groups hold
        // it, so a candidate costs a few operations.
        mx.assign((size_t)most * 4, 0);
        auto rescan = [&](uint32_t n) {
            uint8_t* m4 = &mx[n * 4];
            m4[0] = m4[1] = m4[2] = m4[3] = 0;
            for (int k = 0; k < 16; ++k) {
                const uint8_t a = ha[n * 16 + k], b = hb[n * 16 + k];
                if (a > m4[0]) { m4[0] = a; m4[1] = 1; } else if (a == m4[0]) ++m4[1];
                if (b > m4[2]) { m4[2] = b; m4[3] = 1; } else if (b == m4[2]) ++m4[3];
            }
        };
        // fullest count of histogram h (maximum M held by `at` groups) once a lane leaves group p and joins group q
        auto moved = [](const uint8_t* h, int M, int at, int p, int q) {
            if (p == q) return M;
            if (h[q] + 1 > M) return h[q] + 1;
            return (h[p] == M && at == 1 && h[q] + 1 < M) ? M - 1 : M;
        };
        for (uint32_t n = 0; n < most; ++n) rescan(n);
        for (int pass = 0; pass < STREAM_CLIMB; ++pass) {
            bool improved = false;
            for (uint32_t n = 0; n < most; ++n) {
                const uint8_t* an = &ha[n * 16];
                const uint8_t* bn = &hb[n * 16];
                const uint8_t* xn = &mx[n * 4];
                if (xn[0] + xn[2] <= 2) continue;
                for (int l = 0; l < 16; ++l) {
                    if (cnt[l] <= n) continue;
                    const uint32_t e = ent[l][n];
                    const int ae = ga(e), be = gb(e);
                    if (!((an[ae] == xn[0] && xn[0] > 1) || (bn[be] == xn[2] && xn[2] > 1))) continue;
                    int best = 0;
                    uint32_t bm = n;
                    for (uint32_t m = 0; m < cnt[l]; ++m) {
                        if (m == n) continue;
                        const uint32_t f = ent[l][m];
                        const int af = ga(f), bf = gb(f);
                        const uint8_t* am = &ha[m * 16];
                        const uint8_t* bq = &hb[m * 16];
                        const uint8_t* xm = &mx[m * 4];
                        const int clocks = moved(an, xn[0], xn[1], ae, af) + moved(bn, xn[2], xn[3], be, bf) +
                                           moved(am, xm[0], xm[1], af, ae) + moved(bq, xm[2], xm[3], bf, be) -
                                           (xn[0] + xn[2] + xm[0] + xm[2]);
                        if (clocks > 0) continue;
                        int sq = 0;
                        if (af != ae) sq += 4 + 2 * ((int)an[af] - an[ae] + am[ae] - am[af]);
                        if (bf != be) sq += 4 + 2 * ((int)bn[bf] - bn[be] + bq[be] - bq[bf]);
                        const int delta = clocks * 1024 + sq;
                        if (delta < best) { best = delta; bm = m; }
                    }
                    if (bm != n) {
                        const uint32_t f = ent[l][bm];
                        add(n, e, -1); add(bm, f, -1); add(n, f, 1); add(bm, e, 1);
                        std::swap(ent[l][n], ent[l][bm]);
                        rescan(n);
                        rescan(bm);
                        improved = true;
                        if (xn[0] + xn[2] <= 2) break;
                    }
                }
            }
            if (!improved) break;
        }
        // Write the slots back.  A lane that has run out repeats one of its own codewords (from the least used bank
        // group) against one of the 16 chunks of x that are kept at zero (one per bank group).  A lane without a row,
        // or whose row has no entry here, reads what a neighbour reads (the same addresses are one broadcast read); the
        // kernel drops its sum.
        for (uint32_t n = 0; n < ns; ++n) {
            uint32_t chosen[16];
            int donor = -1;
            for (int l = 0; l < 16; ++l)
                if (cnt[l] > n) { chosen[l] = ent[l][n]; if (donor < 0) donor = l; }
            for (int l = 0; l < 16; ++l) {
                if (cnt[l] > n || cnt[l] == 0) continue;
                uint32_t bi = 0;
                for (uint32_t i = 1; i < cnt[l]; ++i)
                    if (ha[n * 16 + ga(ent[l][i])] < ha[n * 16 + ga(ent[l][bi])]) bi = i;
                int kb = 0;
                for (int k = 1; k < 16; ++k)
                    if (hb[n * 16 + k] < hb[n * 16 + kb]) kb = k;
                chosen[l] = (ent[l][bi] & ((1u << STREAM_SLICE_BITS) - 1u)) | ((uint32_t)(zero_chunk + kb) << STREAM_SLICE_BITS);
                add(n, chosen[l], 1);
                if (donor < 0) donor = l;
            }
            for (int l = 0; l < 16; ++l) {
                if (cnt[l] == 0) chosen[l] = donor >= 0 ? chosen[donor] : 0u;
                *rec_of(base, lanes[l], n) = chosen[l];
            }
        }
    }
};

// One step of 64 lanes x eps entries (one per word) into its bytes: 3 bytes per entry (wide), or the three 21-bit
// entries of a lane in one 64-bit word (narrow).
static void encode_step(const uint32_t* e, const StreamFmt& f, unsigned char* out) {
    for (int lane = 0; lane < 64; ++lane) {
        const uint32_t* r = e + (size_t)lane * f.eps;
        unsigned char* o = out + (size_t)lane * f.lane_bytes;
        if (f.narrow) {
            const uint64_t w = (uint64_t)r[0] | (uint64_t)r[1] << 21 | (uint64_t)r[2] << 42;
            for (int b = 0; b < 8; ++b) o[b] = (unsigned char)(w >> (8 * b));
        } else {
            for (int k = 0; k < 4; ++k) { o[3 * k] = (unsigned char)r[k]; o[3 * k + 1] = (unsigned char)(r[k] >> 8); o[3 * k + 2] = (unsigned char)(r[k] >> 16); }
        }
    }
}

int stream_build_host(const uint32_t* tags, int R, int W, int C, int d, int bits, const uint8_t* row_mask, int runs,
                      unsigned char* out, size_t bytes, int* runs_out, int* groups_out, const uint16_t* table, int G,
                      const uint8_t* row_book) {
    StreamPlan P;
    plan_stream(tags, R, W, C, d, bits, row_mask, runs, P, table != nullptr, G, row_book);
    const uint16_t* remap = table ? P.remap.data() : nullptr;
    const StreamGeom& g = P.g;
    const StreamFmt f = g.fmt;
    const uint32_t EPS = (uint32_t)f.eps, PF = (uint32_t)f.pf, FS = (uint32_t)g.fs;
    const size_t need = g.off_steps + (size_t)g.total_steps * f.step_bytes;
    if (g.total_steps >= ((uint64_t)1 << 32) || g.runs >= (1 << 16)) return fail(SQ_EUNSUPPORTED, "sq_stream_build: matrix too large");
    if (bytes < need) return fail(SQ_EINVAL, "sq_stream_build: buffer %zu < %zu", bytes, need);
    memset(out, 0, need);
    memcpy(out, P.head4.data(), P.head4.size() * 4);
    memcpy(out + g.off_runs, P.runs.data(), P.runs.size() * sizeof(StreamRun));
    memcpy(out + g.off_rows, P.base.data(), P.base.size() * 4);
    if (table) {
        uint16_t* tab = (uint16_t*)(out + g.off_table);
        uint16_t* unmap = (uint16_t*)(out + g.off_unmap);
        for (int k = 0; k < (1 << bits); ++k) {
            memcpy(tab + (size_t)remap[k] * d, table + (size_t)k * d, (size_t)d * 2);
            unmap[remap[k]] = (uint16_t)k;
        }
    }
    std::vector<uint32_t> place(R);
    for (size_t k = 0; k < P.base.size(); ++k)
        if (P.base[k] != STREAM_NO_ROW) place[P.base[k]] = (uint32_t)k;
    P.slot32.assign((size_t)g.NV * g.NG * 64, STREAM_NO_ROW);
    uint32_t* slots = P.slot32.data();
    // the steps are made group after group (P.goff), one entry per word, and moved to their places at the end
    std::vector<uint32_t> laid((size_t)P.logical_steps * 64 * EPS, 0);
    uint32_t* steps = laid.data();
    auto rec = [&](size_t step0, uint32_t lane, uint32_t n) { return steps + ((step0 + n / EPS) * 64 + lane) * EPS + n % EPS; };
    parallel_rows(R, [&](int a, int b) {
        std::vector<uint32_t> q(g.NV), last(g.NV);
        for (int r = a; r < b; ++r) {
            const uint32_t* row = tags + (size_t)r * W;
            const uint32_t book = row_book ? (uint32_t)(row_book[r] & (G - 1)) << bits : 0u;
            std::fill(q.begin(), q.end(), 0u);
            std::fill(last.begin(), last.end(), 0u);
            for (int v = 0; v < g.NV; ++v) {
                const uint32_t k = P.pos[(size_t)v * R + r];
                slots[(size_t)v * g.NG * 64 + k] = place[r] | ((uint32_t)P.cnt[(size_t)v * R + r] << STREAM_ROW_BITS);
            }
            for (int j = 0; j < g.U; ++j) {
                uint32_t t = host_tag(row, W, bits, j);
                if (remap) t = remap[t];
                t |= book;
                const int kp = j / g.PC, v = kp * g.NS + (int)(t >> STREAM_SLICE_BITS);
                const uint32_t k = P.pos[(size_t)v * R + r], n = q[v]++;
                const uint32_t e = (t & ((1u << STREAM_SLICE_BITS) - 1u)) | ((uint32_t)(j - kp * g.PC) << STREAM_SLICE_BITS);
                *rec(P.goff[(size_t)v * g.NG + (k >> 6)], k & 63, n) = e;
                last[v] = e & ((1u << STREAM_SLICE_BITS) - 1u);
            }
            // Padding up to the group's longest row: the row's last codeword of the bucket again, at the chunk of x
            // that the kernel keeps at zero, so padding adds exactly nothing and needs no test in the inner loop
            // (a codeword that is not finite is already part of the row's sum; a row without entries in the
            // bucket is dropped by its slot).
            for (int v = 0; v < g.NV; ++v) {
                const uint32_t k = P.pos[(size_t)v * R + r];
                const size_t gi = (size_t)v * g.NG + (k >> 6);
                const uint32_t cap = (P.goff[gi + 1] - P.goff[gi]) * EPS;
                const uint32_t e = last[v] | ((uint32_t)g.PC << STREAM_SLICE_BITS);
                for (uint32_t n = q[v]; n < cap; ++n) *rec(P.goff[gi], k & 63, n) = e;
            }
        }
    });
    // Second pass, group by group: the order of a lane's entries is free (padding stays behind them), so it is
    // chosen to keep the LDS gathers apart.  A 16-byte LDS read of a wave takes four clocks of 16 lanes each
    // (LDS_CLOCK_LANES), and two lanes of a clock collide when their addresses differ but fall into the same group
    // of four banks (address / 16 mod 16): BankMatch arranges the entries of each clock's lanes.
    parallel_rows(g.NV * g.NG, [&](int a, int b) {
        BankMatch bm;
        bm.eps = EPS;
        for (int vg = a; vg < b; ++vg) {
            const uint32_t st0 = P.goff[vg], ns = (P.goff[vg + 1] - st0) * EPS;
            if (ns == 0) continue;
            const uint32_t* sl = slots + (size_t)vg * 64;
            uint32_t* base = steps + (size_t)st0 * 64 * EPS;
            for (int q = 0; q < 4; ++q) bm.order_lanes(base, sl, LDS_CLOCK_LANES[q], ns, (uint32_t)g.PC);
        }
    });
    // to their places: the first FS steps of every unit into the first-steps region, the rest behind each other; and
    // the slots in their 16-bit form (place counted from the run's first place, entries or none)
    uint16_t* slot16 = (uint16_t*)(out + g.off_slots);
    parallel_rows(g.NV * g.NG, [&](int a, int b) {
        for (int vg = a; vg < b; ++vg) {
            const uint32_t* h = &P.head4[(size_t)vg * 4];
            const int v = vg / g.NG, nst = (int)h[1], split = (int)(h[3] & 0xFFu);
            const uint32_t p0 = (h[3] >> 8) * 64u;
            for (int lane = 0; lane < 64; ++lane) {
                const uint32_t s32 = slots[(size_t)vg * 64 + lane];
                slot16[(size_t)vg * 64 + lane] = (s32 & STREAM_NO_ROW) == STREAM_NO_ROW
                    ? (uint16_t)STREAM_SLOT_NONE
                    : (uint16_t)(((s32 & STREAM_NO_ROW) - p0) | ((s32 >> STREAM_ROW_BITS) ? STREAM_SLOT_HAS : 0u));
            }
            const uint32_t* src = steps + (size_t)P.goff[vg] * 64 * EPS;
            for (int j = 0; j < split; ++j) {
                const int s0 = nst * j / split, s1 = nst * (j + 1) / split;
                for (int t = s0; t < s1; ++t) {
                    const uint64_t to = (uint32_t)(t - s0) < PF ? ((uint64_t)(h[2] + j) * g.NV + v) * FS + (t - s0)
                                                                 : (uint64_t)h[0] + t - (uint64_t)PF * (j + 1);
                    encode_step(src + (size_t)t * 64 * EPS, f, out + g.off_steps + to * f.step_bytes);
                }
            }
        }
    });
    if (runs_out) *runs_out = g.runs | (P.GR << 16) | ((P.orders_max - 1) << 24) | ((g.fs - 1) << 27) | (table ? STREAM_BALANCED : 0);
    if (groups_out) *groups_out = g.NG;
    return SQ_OK;
}

// ---------------------------------------------------------------------------------------- device

struct StreamPiece {
    const unsigned char* stream;
    const uint16_t* table;
    const uint16_t* row_scale;
    float* part;                      // [NV][NB][NG * 64] words, indexed by place: zero before the launch, zero after it
    const int32_t* perms;             // [M, C] column orders or NULL
    int R, C, U, NS, NV, PC, NG, y_off;
    int fs;                           // steps per unit in the first-steps region
    uint32_t off_slots, off_runs, off_rows, off_steps;
    int wg_begin, nwg;                // first workgroup of the piece; workgroups (= runs) per bucket
};

struct StreamArgs {
    StreamPiece p[GEMV_MAX_PIECES_STREAM];
    int n;
    const uint16_t* x;                // activation row b0
    void* y;                          // output row b0
    int64_t ldx, ldy;
    int nb;                           // activation rows of this pass (<= NB)
    int xs;                           // LDS bytes of one activation row's part of x (its chunks + 16 zero chunks)
    int xcopies;                      // copies of x per activation row in LDS: the most column orders in one run of the launch
    int xtmp;                         // bytes per activation row of its copy in natural order in LDS (column orders are then
                                      // applied from LDS), 0: gathered from memory
    int orders;                       // 1: some piece has column orders
    int narrow;                       // 1: the pieces' entries are 21 bits wide (StreamF<1>)
    int xtmp_own;                     // 1: those copies have LDS of their own behind everything else, 0: they sit where the slice goes
    int nl_max;                       // places of the longest run (64 per group): floats per row of the LDS partial sums
    int x_dtype, y_dtype;
    // Producer of the activation row (stream_kernel<1, NX, 1> only): the row is computed while it is staged instead
    // of being read from x: round(v * rsqrt(mean(v^2) + eps) * w) with v = h_in + add.  add / w / x_out hold x_dtype;
    // x_out (and h_out) are written once per launch.  (SiLU(gate) * up is not produced this way: every workgroup
    // would evaluate the whole row's exponentials, several microseconds against a stand-alone launch of under four.)
    const float* h_in;
    float* h_out;
    const uint16_t* add;
    const uint16_t* w;
    uint16_t* x_out;
    float eps;
    // Consumer of the output (pieces 0 and 1 = the gate and the up projection, same shape, no column orders): instead of
    // y the launch writes act[b * ld_act + r] = silu(round(Y[b, r])) * round(Y[b, R + r]) in y_dtype, the arithmetic of
    // silu_mul_kernel on the rounded outputs.  NULL: y is written.
    uint16_t* act;
    int64_t ld_act;
    uint32_t* err;                    // the workspace header's error word (SQ_WS_ERR_OFF)
    uint32_t* host_err;               // its host-visible copy (pinned host memory) or NULL
    int spin_max;                     // polls of an item's partial sums before it gives up
};

// The operands of one chunk (8 elements) of the produced row, fetched first and finished once the row's scale is known.
// h, lo = add, hi = w.
struct ProRaw { float h[8]; uint32_t lo[4], hi[4]; };

// chunk ci in natural order: 16-byte loads (every pointer 16-byte aligned)
template <int PRO>
__device__ __forceinline__ ProRaw pro_fetch(const StreamArgs& a, int ci) {
    ProRaw r;
    const u32x4 hi = reinterpret_cast<const u32x4*>(a.w)[ci];
    u32x4 lo = u32x4{0u, 0u, 0u, 0u};
    if (a.add) lo = reinterpret_cast<const u32x4*>(a.add)[ci];
#pragma unroll
    for (int k = 0; k < 4; ++k) { r.lo[k] = lo[k]; r.hi[k] = hi[k]; }
    if (PRO == 1) {
        const float4v h0 = reinterpret_cast<const float4v*>(a.h_in)[2 * ci], h1 = reinterpret_cast<const float4v*>(a.h_in)[2 * ci + 1];
#pragma unroll
        for (int k = 0; k < 4; ++k) { r.h[k] = h0[k]; r.h[4 + k] = h1[k]; }
    }
    return r;
}
__device__ __forceinline__ float pro_f(uint32_t pair, int k, int dtype) {
    const uint16_t b = (uint16_t)(pair >> (16 * (k & 1)));
    return dtype == SQ_BF16 ? bf2f(b) : h2f(b);
}
// v = h + add of element k of a fetched chunk (PRO 1)
__device__ __forceinline__ float pro_v(const StreamArgs& a, const ProRaw& r, int k) {
    return a.add ? r.h[k] + pro_f(r.lo[k >> 1], k, a.x_dtype) : r.h[k];
}
template <int PRO>
__device__ __forceinline__ u32x4 pro_finish(const StreamArgs& a, const ProRaw& r, float rstd) {
    uint32_t e[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        e[k] = round16(pro_v(a, r, k) * rstd * pro_f(r.hi[k >> 1], k, a.x_dtype), a.x_dtype);
    }
    return u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
}

constexpr int STREAM_TAB = 65536;     // the codebook slice
constexpr uint32_t STREAM_ZERO_SUM = 0x7FFFFFFFu;  // how a partial sum with all bits zero is written (zero = not there yet)
constexpr int STREAM_SPIN_MAX = 1 << 18;           // polls of an item's partial sums before it gives up (default)

// LDS bytes of one activation row's part of x: pc chunks plus 16 zero chunks (one per bank group); the narrow format
// gives every copy 8 KB, so the address of a chunk is its offset OR-ed into the copy's base
static inline int stream_xs(int pc) { return stream_fmt(pc).narrow ? 8192 : (pc + 16) * 16; }

// what a wave walks of a group: nst steps, of which step t >= PF is step rb + t of the buffer (the first PF are in the
// first-steps region), and this lane's slot
struct StreamHead { uint32_t rb; int nst; uint32_t slot; };
// a group's words as loaded ({rest, nst, unit0, split | g0 << 8} and this lane's slot) and its index in the run
struct StreamHeadRaw { uint32_t rest, nst, sl; int k; };

// Bit field [OFF, OFF + W) of v times 16, plus base: the LDS address of a chunk of x from the word that holds its
// index, in two instructions (v_bfe_u32, v_lshl_add_u32).  Written as a shift, a mask and an addition the compiler
// makes three of it.
template <int OFF, int W>
__device__ __forceinline__ uint32_t stream_field16(uint32_t v, uint32_t base) {
    uint32_t f, r;
    asm("v_bfe_u32 %0, %1, %2, %3" : "=v"(f) : "v"(v), "n"(OFF), "n"(W));
    asm("v_lshl_add_u32 %0, %1, 4, %2" : "=v"(r) : "v"(f), "v"(base));
    return r;
}

// The entry format as the kernels see it (sq_stream.h: StreamFmt).  addrs(): the LDS byte addresses of every entry's
// codeword (its tag times 16: the slice begins at LDS address 0) and of its chunk of x (times 16, plus xbase), four
// instructions per entry (five for one of the wide ones).
template <int NAR> struct StreamF;
template <> struct StreamF<0> {
    static constexpr int EPS = 4, LB = 12, SB = 768, PF = 3;
    static constexpr uint32_t CMASK = 0xFFFu;
    typedef u32x3 vec;
    // (bits above an entry's 24 are left in place: the address fields are cut out where they are used)
    static __device__ __forceinline__ void entries(const vec& c, uint32_t* e) {
        e[0] = c.x; e[1] = (c.x >> 24) | (c.y << 8); e[2] = (c.y >> 16) | (c.z << 16); e[3] = c.z >> 8;
    }
    static __device__ __forceinline__ void addrs(const vec& c, uint32_t xbase, uint32_t* ta, uint32_t* xa) {
        ta[0] = (c.x << 4) & 0xFFF0u;                               xa[0] = stream_field16<12, 12>(c.x, xbase);
        ta[1] = __builtin_amdgcn_alignbit(c.y, c.x, 20) & 0xFFF0u;  xa[1] = stream_field16<4, 12>(c.y, xbase);
        ta[2] = (c.y >> 12) & 0xFFF0u;                              xa[2] = stream_field16<0, 12>(__builtin_amdgcn_alignbit(c.z, c.y, 28), xbase);
        ta[3] = (c.z >> 4) & 0xFFF0u;                               xa[3] = stream_field16<20, 12>(c.z, xbase);
    }
    static __device__ __forceinline__ vec zero() { return vec{0u, 0u, 0u}; }
};
template <> struct StreamF<1> {
    static constexpr int EPS = 3, LB = 8, SB = 512, PF = 4;
    static constexpr uint32_t CMASK = 0x1FFu;
    typedef u32x2 vec;
    static __device__ __forceinline__ void entries(const vec& c, uint32_t* e) {
        e[0] = c.x; e[1] = (c.x >> 21) | (c.y << 11); e[2] = c.y >> 10;
    }
    static __device__ __forceinline__ void addrs(const vec& c, uint32_t xbase, uint32_t* ta, uint32_t* xa) {
        ta[0] = (c.x << 4) & 0xFFF0u;                               xa[0] = stream_field16<12, 9>(c.x, xbase);
        ta[1] = __builtin_amdgcn_alignbit(c.y, c.x, 17) & 0xFFF0u;  xa[1] = stream_field16<1, 9>(c.y, xbase);
        ta[2] = (c.y >> 6) & 0xFFF0u;                               xa[2] = stream_field16<22, 9>(c.y, xbase);
    }
    static __device__ __forceinline__ vec zero() { return vec{0u, 0u}; }
};

// Optional per-wave timeline (debug builds define SQ_TRACE_POINT).
#ifndef SQ_TRACE_POINT
#define SQ_TRACE_POINT(k)
#endif
#ifndef SQ_TRACE_DEP
#define SQ_TRACE_DEP(k, reg, v)         // a point taken once value v (in a "s" or "v" register) has arrived
#endif

// s_waitcnt immediate that waits until at most n vector-memory operations are outstanding and leaves the other
// counters alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8)
constexpr int stream_vmcnt_only(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

typedef const __attribute__((address_space(1))) void* stream_gptr_t;
typedef __attribute__((address_space(3))) void* stream_lptr_t;
typedef __attribute__((address_space(3))) u32x4 stream_lds_u32x4;

// NB activation rows per pass (every entry's codeword is gathered once and multiplied with NB x chunks), NX chunks of
// a row's part of x per thread (1: parts of up to 1024 chunks, 4: up to 4096), NAR: the entry format (1: 21-bit entries,
// parts of at most 496 chunks).  One workgroup of 16 waves per CU.
// LDS: [codebook slice 64 KB][NB x parts of a.xs bytes][partial sums of the run: NB x a.nl_max floats][two words of flags]
// [16 block sums (PRO 1)].
template <int NB, int NX, int PRO = 0, int ORD = 1, int NAR = 0>
__global__ __launch_bounds__(STREAM_NW * 64) void stream_kernel(StreamArgs a) {
    static_assert(PRO == 0 || (PRO == 1 && NB == 1 && ORD == 0), "produced activations: add + norm, one row, no column orders");
    typedef StreamF<NAR> F;
    typedef typename F::vec evec;
    constexpr int STREAM_PF = F::PF;
    constexpr int NW = STREAM_NW, NTH = NW * 64;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int pi = 0;
#pragma unroll
    for (int k = 1; k < GEMV_MAX_PIECES_STREAM; ++k)
        if (k < a.n && (int)blockIdx.x >= a.p[k].wg_begin) pi = k;
    const StreamPiece P = a.p[pi];                             // by value: the piece's fields arrive in one batch of scalar loads
    // ORD 0: no piece of the launch has column orders (everything that serves them compiles away)
    const int32_t* const perms = ORD ? P.perms : nullptr;
    SQ_TRACE_DEP(7, "s", P.NV);
    // Workgroups go to the 8 XCDs in turn (workgroup i to XCD i mod 8), each with an L2 of its own.  When the
    // bucket count is a multiple of 8 the bucket (and with it the slice) is made a function of the workgroup index
    // modulo 8, so an XCD only ever stages an eighth of the buckets' slices (one fetch from memory, then hits in
    // its L2).  Either way the NV workgroups of a run are consecutive in the grid: they wait for each other's partial
    // sums at the end, and workgroups are dispatched in grid order, so whoever a workgroup waits for is running or done.
    const int local = (int)blockIdx.x - P.wg_begin;
    int v, wi;
    if ((P.NV & 7) == 0 && (P.wg_begin & 7) == 0) {
        const int per = P.NV >> 3, rest = local >> 3;           // buckets per XCD; index among that XCD's workgroups
        v = (local & 7) + 8 * (rest % per);
        wi = rest / per;
    } else {
        wi = local / P.NV;
        v = local - wi * P.NV;
    }
    const int s = v % P.NS, kp = v / P.NS;
    SQ_TRACE_POINT(0);
    // this workgroup's run: groups g0 .. g0 + ng - 1 of the bucket, all of one column order
    // (without column orders every run but the last has ceil(NG / runs) groups: no need to wait for the table)
    const int32_t* run = reinterpret_cast<const int32_t*>(P.stream + P.off_runs) + wi * 8;
    const int gr = (P.NG + P.nwg - 1) / P.nwg;
    const int g0 = perms ? run[0] : wi * gr, ng = min(perms ? run[1] : min(gr, P.NG - g0), a.nl_max >> 6);
    // the run's column orders (with row orders only): copy i of x, gathered through order i, serves the groups from
    // bound i on
    const int no = perms ? min(max(run[2], 1), a.xcopies) : 1;
    const uint32_t bnd_lo = perms ? (uint32_t)run[4] : 0u, bnd_hi = perms ? (uint32_t)run[5] : 0u;
    const uint32_t ord_lo = perms ? (uint32_t)run[6] : 0u, ord_hi = perms ? (uint32_t)run[7] : 0u;
    auto byte_of = [](uint32_t lo, uint32_t hi, int i) { return (int)(((i < 4 ? lo >> (8 * i) : hi >> (8 * (i - 4)))) & 0xFFu); };

    const u32x4* gw = reinterpret_cast<const u32x4*>(P.stream) + (size_t)v * P.NG + g0;   // {rest, nst, unit0, split} per group
    const int u0 = perms ? run[3] : wi * gr * stream_split_of(gr);   // this run's first unit
    const uint16_t* slots = reinterpret_cast<const uint16_t*>(P.stream + P.off_slots) + ((size_t)v * P.NG + g0) * 64;
    const unsigned char* steps = P.stream + P.off_steps + lane * F::LB;
    const size_t np = (size_t)P.NG * 64;
    float* part = P.part + (size_t)v * NB * np;
    const int xs = a.xs;
    // (the inner loop forms LDS addresses as numbers counted from the start of the dynamic LDS: that is address 0 in a
    // kernel without static LDS; a build in which it is not leaves y unwritten, which no test survives)
    if ((uint32_t)(uintptr_t)(stream_lptr_t)lds != 0u) return;
    float* psum = reinterpret_cast<float*>(lds + STREAM_TAB + a.xcopies * NB * xs);   // [NB][a.nl_max], indexed by place in the run
    unsigned* flag = reinterpret_cast<unsigned*>(psum + (size_t)NB * a.nl_max);  // [1] next group

    // The groups of a run are sorted longest first.  Wave w starts with group w, then group 2 NW - 1 - w; after
    // that every wave draws the next unclaimed group from a counter in LDS, so all waves stay busy to the end.
    // The head of a group (its first step, its step count, the lane's row and count) is fetched one group
    // ahead; the first one goes out before the staging loads.
    // A run with at most NW / 2 groups would leave waves idle while the others walk their steps a few fetches at
    // a time; there `split` = 16 / groups waves share a group, each takes a contiguous share of its steps, and
    // the shares are added in wave order through LDS.  The share count follows from the group count alone, so a
    // row's sums are formed in the same order whatever NB, NX and PRO are.
    const int split = ng * 2 <= NW ? NW / ng : 1;
    const int sub = wave % split;
    // What this wave walks of group k, from the group's loaded words: the whole group, or its share of the steps.
    auto head_from = [&](int k, uint32_t rest, uint32_t nst_g, uint32_t sl) {
        StreamHead h{rest - (uint32_t)STREAM_PF, (int)nst_g, sl};
        if (k >= ng) h = StreamHead{0u, 0, STREAM_SLOT_NONE};
        else if (split > 1) {                                   // uniform in the workgroup
            // (a share that holds only padding of a row adds exactly nothing, like padding anywhere else)
            const int s0 = h.nst * sub / split, s1 = h.nst * (sub + 1) / split;
            h.rb = rest + (uint32_t)s0 - (uint32_t)(STREAM_PF * (sub + 1));
            h.nst = s1 - s0;
        }
        return h;
    };
    // (loads without a branch around them, from a clamped index: the compiler then knows how many loads are in
    // flight and later waits do not have to cover these.)  The group's words are the same in every lane; loaded
    // through an index the compiler takes for a per-lane value they stay in vector registers, and they are kept as
    // loaded (`head_raw`) until the group is started (`resolve`): nothing waits for them where they are requested.
    // A load the compiler knows to be uniform, or whose result is used at once, is followed by a wait there: one
    // memory round trip of standstill per group.
    auto uni = [](int v) { return (int)__builtin_amdgcn_readfirstlane(v); };
    auto head_raw = [&](int k) {
        int kc = min(k, ng - 1);
        asm volatile("" : "+v"(kc));
        const u32x2 w = *reinterpret_cast<const u32x2*>(gw + kc);       // (only the first two of the four words: every register
                                                                        // a load writes must stay in use until it has landed)
        return StreamHeadRaw{w.x, w.y, (uint32_t)slots[(size_t)kc * 64 + lane], k};
    };
    // (the empty asm pins the arithmetic to the place of the call: hoisted to where the words are loaded it would bring
    // the wait along)
    auto resolve = [&](StreamHeadRaw r) {
        asm volatile("" : "+v"(r.rest), "+v"(r.nst), "+v"(r.sl));
        return head_from(r.k, r.rest, r.nst, r.sl);
    };
    // The first STREAM_PF steps of this wave's unit of group k: their place follows from indices alone, so they are
    // requested without having read anything (every unit has STREAM_PF steps there, used or not).
    const int fs = P.fs;
    auto first_steps = [&](int k, evec* nx) {
        const int unit = u0 + min(k, ng - 1) * split + sub;
        const unsigned char* en = steps + ((size_t)unit * P.NV + v) * (size_t)(fs * F::SB);
#pragma unroll
        for (int q = 0; q < STREAM_PF; ++q) nx[q] = *reinterpret_cast<const evec*>(en + (size_t)min(q, fs - 1) * F::SB);
    };
    // The error word of the exchange, requested now and looked at when y is written: once a launch on this workspace
    // has given up waiting, partial sums may have arrived late and the header may be dirty; every launch then writes
    // NaN until the host has reset the workspace.
    const uint32_t err0 = __hip_atomic_load(a.err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    int kcur = wave, knext = 2 * NW - 1 - wave;
    if (split > 1) {                                            // one share of one group per wave, or nothing
        kcur = wave < ng * split ? wave / split : ng;
        knext = ng;
    }
    // Column orders through LDS (a.xtmp > 0): the activation rows first sit in natural order where the slice goes, and
    // the kd 16 KB blocks of the slice that they cover are copied once the rows have been read from there.
    const bool via_lds = PRO == 0 && perms != nullptr && a.xtmp > 0;   // uniform in the workgroup
    const int kd = via_lds && !a.xtmp_own ? (NB * a.xtmp + NTH * 16 - 1) / (NTH * 16) : 0;
    // The first head's words are requested first of all (through a vector index, see `head`): vector loads come back in
    // the order they were issued, and behind the 64 KB of slice these three words would arrive a bulk copy later, with
    // the first steps, whose addresses they give, another round trip behind.  They are used once the slice copy and
    // the loads of x have gone out.
    int kc0 = min(kcur, ng - 1);
    asm volatile("" : "+v"(kc0));
    const u32x2 head_w = *reinterpret_cast<const u32x2*>(gw + kc0);
    const uint32_t head_s = slots[(size_t)kc0 * 64 + lane];
    __builtin_amdgcn_sched_barrier(0);
    // The codebook slice is copied global -> LDS without passing through registers (a wave instruction moves 1 KB, lane l
    // to the wave's base + 16 l).
    {
        const unsigned char* src = reinterpret_cast<const unsigned char*>(P.table) + (size_t)s * STREAM_TAB;
#pragma unroll
        for (int k = 0; k < STREAM_TAB / (NTH * 16); ++k)
            if (k >= kd)
                __builtin_amdgcn_global_load_lds((stream_gptr_t)(src + ((size_t)k * NTH + tid) * 16),
                                                 (stream_lptr_t)(lds + (k * NTH + wave * 64) * 16), 16, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    StreamHeadRaw hn;
    evec nx[STREAM_PF];
#pragma unroll
    for (int q = 0; q < STREAM_PF; ++q) nx[q] = F::zero();

    // Stage this part of the NB activation rows (as fp16); the first group's steps are requested before anything waits
    // for the staging loads.
    {
        u32x4 xq[NB][NX];
        const int c0 = kp * P.PC, nc = min(P.PC, P.U - c0);
        // this thread's items of the staged x: item it = (copy, chunk) = (it / nc, it % nc), it = tid + k * NTH
        const int total = no * nc;
        int it_o[NX], it_c[NX];
#pragma unroll
        for (int k = 0; k < NX; ++k) {
            const int it = min(tid + k * NTH, total - 1);
            it_o[k] = no > 1 ? it / nc : 0;
            it_c[k] = it - it_o[k] * nc;
        }
        if (PRO != 0) {
            // every operand of the produced row is requested before anything waits: this thread's chunks, then
            // (PRO 1) its share of the whole row for the mean square
            ProRaw raw[NX];
#pragma unroll
            for (int k = 0; k < NX; ++k) raw[k] = pro_fetch<PRO>(a, c0 + it_c[k]);
            float rstd = 0.f;
            if (PRO == 1) {
                // Mean square of the whole row in the stand-alone kernel's order, so both give the same bits: slot j
                // of 1024 (= thread j) adds the squares of chunks j, j + 1024, ... element by element with fused
                // multiply-adds, each block of 64 slots is folded by the wave butterfly, the 16 block sums are added in
                // turn.
                static_assert(NTH == 1024, "one slot per thread");
                float* red = reinterpret_cast<float*>(flag + 4);
                float ps = 0.f;
                if (nc == P.U && P.U <= NX * NTH) {
                    // one column part, natural order: this thread's chunks are its slot's chunks, already fetched
#pragma unroll
                    for (int k = 0; k < NX; ++k)
                        if (tid + k * NTH < P.U) {
#pragma unroll
                            for (int e = 0; e < 8; ++e) { const float vv = pro_v(a, raw[k], e); ps = __builtin_fmaf(vv, vv, ps); }
                        }
                } else if (P.U <= NTH) {                        // one chunk per slot
                    const ProRaw r1 = pro_fetch<1>(a, min(tid, P.U - 1));
                    if (tid < P.U) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) { const float vv = pro_v(a, r1, e); ps = __builtin_fmaf(vv, vv, ps); }
                    }
                } else {
                    for (int c = tid; c < P.U; c += NTH) {
                        const ProRaw r = pro_fetch<1>(a, c);
#pragma unroll
                        for (int e = 0; e < 8; ++e) { const float vv = pro_v(a, r, e); ps = __builtin_fmaf(vv, vv, ps); }
                    }
                }
                ps = wave_sum(ps);
                if (lane == 0) red[wave] = ps;
                __syncthreads();
                float tot = 0.f;
#pragma unroll
                for (int q = 0; q < NW; ++q) tot += red[q];
                rstd = rsqrtf(tot / (float)P.C + a.eps);
            }
#pragma unroll
            for (int k = 0; k < NX; ++k) xq[0][k] = pro_finish<PRO>(a, raw[k], rstd);
            if (pi == 0 && s == 0 && wi == 0) {
                // one workgroup per column part leaves the produced row (and the updated residual) in memory
#pragma unroll
                for (int k = 0; k < NX; ++k) {
                    const int c = tid + k * NTH;
                    if (c >= nc) continue;
                    reinterpret_cast<u32x4*>(a.x_out)[c0 + c] = xq[0][k];
                    if (PRO == 1 && a.h_out) {
                        float4v o0, o1;
#pragma unroll
                        for (int e = 0; e < 4; ++e) { o0[e] = pro_v(a, raw[k], e); o1[e] = pro_v(a, raw[k], 4 + e); }
                        reinterpret_cast<float4v*>(a.h_out)[2 * (c0 + c)] = o0;
                        reinterpret_cast<float4v*>(a.h_out)[2 * (c0 + c) + 1] = o1;
                    }
                }
            }
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const uint16_t* xr = a.x + (int64_t)min(b, a.nb - 1) * a.ldx;
            if (PRO != 0) {
                // filled above
            } else if (perms == nullptr) {
                const u32x4* xsrc = reinterpret_cast<const u32x4*>(xr) + c0;
#pragma unroll
                for (int k = 0; k < NX; ++k) xq[b][k] = xsrc[min(tid + k * NTH, nc - 1)];
            } else if (a.xtmp > 0) {
                // column orders, the row in natural order first: its chunks go to LDS below and the copies are
                // gathered from there (one part per row here, so the row has at most NX * NTH chunks)
                const u32x4* xsrc = reinterpret_cast<const u32x4*>(xr);
#pragma unroll
                for (int k = 0; k < NX; ++k) xq[b][k] = xsrc[min(tid + k * NTH, P.U - 1)];
            } else {
                // chunk j of a row with column order m multiplies x[perm_m[8 j .. 8 j + 7]]
#pragma unroll
                for (int k = 0; k < NX; ++k) {
                    if (k > 0 && tid + k * NTH >= total) { xq[b][k] = xq[b][0]; continue; }
                    const int32_t* pk = perms + (size_t)byte_of(ord_lo, ord_hi, it_o[k]) * P.C + (size_t)(c0 + it_c[k]) * 8;
                    const u32x4 i0 = *reinterpret_cast<const u32x4*>(pk), i1 = *reinterpret_cast<const u32x4*>(pk + 4);
                    const uint32_t e0 = xr[i0.x], e1 = xr[i0.y], e2 = xr[i0.z], e3 = xr[i0.w];
                    const uint32_t e4 = xr[i1.x], e5 = xr[i1.y], e6 = xr[i1.z], e7 = xr[i1.w];
                    xq[b][k] = u32x4{e0 | (e1 << 16), e2 | (e3 << 16), e4 | (e5 << 16), e6 | (e7 << 16)};
                }
            }
        }
        // Column orders through LDS: a scattered 2-byte read from memory occupies the address unit for a clock per lane
        // (8 reads per chunk and copy: microseconds once a run has several orders), the same read from LDS costs a few
        // clocks per wave.  The positions come from memory meanwhile.
        u32x4 ix[NX][2];
        if (via_lds) {
#pragma unroll
            for (int k = 0; k < NX; ++k) {
                const int32_t* pk = perms + (size_t)byte_of(ord_lo, ord_hi, it_o[k]) * P.C + (size_t)(c0 + it_c[k]) * 8;
                ix[k][0] = *reinterpret_cast<const u32x4*>(pk);
                ix[k][1] = *reinterpret_cast<const u32x4*>(pk + 4);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        SQ_TRACE_DEP(8, "v", head_s);
        hn = StreamHeadRaw{head_w.x, head_w.y, head_s, kcur};
        first_steps(kcur, nx);
        __builtin_amdgcn_sched_barrier(0);
        SQ_TRACE_DEP(9, "v", xq[0][0].x);
        if (via_lds) {
            unsigned char* tmp = a.xtmp_own ? reinterpret_cast<unsigned char*>(flag + 20) : lds;   // [NB][a.xtmp]
#pragma unroll
            for (int b = 0; b < NB; ++b) {
#pragma unroll
                for (int k = 0; k < NX; ++k)
                    if (tid + k * NTH < P.U) reinterpret_cast<u32x4*>(tmp + b * a.xtmp)[tid + k * NTH] = xq[b][k];
            }
            __syncthreads();
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const uint16_t* xt = reinterpret_cast<const uint16_t*>(tmp + b * a.xtmp);
#pragma unroll
                for (int k = 0; k < NX; ++k) {
                    if (tid + k * NTH >= total) continue;
                    const u32x4 i0 = ix[k][0], i1 = ix[k][1];
                    const uint32_t e0 = xt[i0.x], e1 = xt[i0.y], e2 = xt[i0.z], e3 = xt[i0.w];
                    const uint32_t e4 = xt[i1.x], e5 = xt[i1.y], e6 = xt[i1.z], e7 = xt[i1.w];
                    xq[b][k] = u32x4{e0 | (e1 << 16), e2 | (e3 << 16), e4 | (e5 << 16), e6 | (e7 << 16)};
                }
            }
            if (kd > 0) __syncthreads();                        // every wave has what it reads of the rows: the slice may land
            const unsigned char* src = reinterpret_cast<const unsigned char*>(P.table) + (size_t)s * STREAM_TAB;
#pragma unroll
            for (int k = 0; k < STREAM_TAB / (NTH * 16); ++k)
                if (k < kd)
                    __builtin_amdgcn_global_load_lds((stream_gptr_t)(src + ((size_t)k * NTH + tid) * 16),
                                                     (stream_lptr_t)(lds + (k * NTH + wave * 64) * 16), 16, 0, 0);
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) {
#pragma unroll
            for (int k = 0; k < NX; ++k) {
                u32x4 q = xq[b][k];
                if (a.x_dtype == SQ_BF16) { q.x = bf2h_x2(q.x); q.y = bf2h_x2(q.y); q.z = bf2h_x2(q.z); q.w = bf2h_x2(q.w); }
                // copy o of activation row b lives at [o][b]
                if (tid + k * NTH < total) reinterpret_cast<u32x4*>(lds + STREAM_TAB + (it_o[k] * NB + b) * xs)[it_c[k]] = q;
            }
        }
        if (tid < no * NB * 16)                                  // the chunks that padding entries multiply with, in every copy
            reinterpret_cast<u32x4*>(lds + STREAM_TAB + (tid >> 4) * xs)[P.PC + (tid & 15)] = u32x4{0u, 0u, 0u, 0u};
        if (tid == 0) flag[1] = 2 * NW;
        // the slice copies were issued before everything except the STREAM_PF loads of the first steps (or last of all)
        if (kd > 0) __builtin_amdgcn_s_waitcnt(stream_vmcnt_only(0));
        else __builtin_amdgcn_s_waitcnt(stream_vmcnt_only(STREAM_PF));
        SQ_TRACE_POINT(10);
    }
    __syncthreads();
    SQ_TRACE_POINT(1);

    float acc_share[NB];                                        // split > 1: this wave's share of its group
    int k_share = -1;
#pragma unroll
    for (int b = 0; b < NB; ++b) acc_share[b] = 0.f;
    while (kcur < ng) {
        const StreamHead h = resolve(hn);
        hn = head_raw(knext);
        int kafter = ng;
        if (knext < ng) {
            unsigned tk = 0;
            if (lane == 0) tk = __hip_atomic_fetch_add(flag + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            kafter = (int)__builtin_amdgcn_readfirstlane(tk);
        }
        const int nst = uni(h.nst);
        const bool has = (h.slot & STREAM_SLOT_HAS) != 0u;
        const uint32_t row = h.slot & STREAM_SLOT_NONE;        // place in the run
        const unsigned char* eb = steps + (size_t)(uint32_t)uni((int)h.rb) * F::SB;
        // the copy of x for this group's column order
        int xc = 0;
#pragma unroll
        for (int oi = 1; oi < STREAM_RUN_ORDERS; ++oi) xc += (oi < no && kcur >= byte_of(bnd_lo, bnd_hi, oi)) ? 1 : 0;
        // LDS byte address of this group's copy of x, kept in a vector register: a chunk's address is then one
        // shift-and-add (the instruction takes one scalar or constant operand, and the shift count is one already)
        uint32_t xbase = (uint32_t)STREAM_TAB + (uint32_t)(xc * NB * xs);
        asm volatile("" : "+v"(xbase));
        // (The same products on the matrix cores, which work beside the vector ALU - v_mfma_f32_4x4x4_16b_f16 gives lane j
        // of every four the dot product of its own four halves of A and B as element j of its result - measured no
        // faster on the large launches and slower on gate|up: 19.2-20.2 against 18.0-18.9 us on one machine.)
        float acc[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[b] = 0.f;
        for (int t0 = 0; t0 < nst; t0 += STREAM_PF) {
            evec cur[STREAM_PF];
#pragma unroll
            for (int q = 0; q < STREAM_PF; ++q) cur[q] = nx[q];
            if (t0 + STREAM_PF < nst) {                         // wave-uniform
#pragma unroll
                for (int q = 0; q < STREAM_PF; ++q)
                    nx[q] = *reinterpret_cast<const evec*>(eb + (size_t)min(t0 + STREAM_PF + q, nst - 1) * F::SB);
            } else {
                if (knext < ng) first_steps(knext, nx);         // the next group's first steps
            }
#pragma unroll
            for (int q = 0; q < STREAM_PF; ++q) {
                if (t0 + q >= nst) break;                       // wave-uniform
                uint32_t ta[F::EPS], xa[F::EPS];
                F::addrs(cur[q], xbase, ta, xa);
                // the LDS reads of EB entries go out together, then their products: a wave does not sit out one
                // LDS round trip per entry
                constexpr int EB = NB == 1 ? F::EPS : NB == 2 ? (NAR ? 3 : 2) : 1;
#pragma unroll
                for (int j0 = 0; j0 < F::EPS; j0 += EB) {
                    u32x4 cw[EB], xv[EB][NB];
#pragma unroll
                    for (int jj = 0; jj < EB; ++jj) {
                        // (LDS addresses as plain numbers: the kernel's dynamic LDS begins at address 0, checked at its
                        // start, and `lds + offset` would cost an addition of that zero per read)
                        cw[jj] = *reinterpret_cast<const stream_lds_u32x4*>((uintptr_t)ta[j0 + jj]);
#pragma unroll
                        for (int b = 0; b < NB; ++b)
                            xv[jj][b] = *reinterpret_cast<const stream_lds_u32x4*>((uintptr_t)(xa[j0 + jj] + (uint32_t)(b * (NAR ? 8192 : xs))));
                    }
#pragma unroll
                    for (int jj = 0; jj < EB; ++jj) {
#pragma unroll
                        for (int b = 0; b < NB; ++b) {
#pragma unroll
                            for (int hh = 0; hh < 4; ++hh) {
                                const uint32_t cwh = cw[jj][hh], xvh = xv[jj][b][hh];  // bit_cast straight from a vector element misreads it
                                acc[b] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, cwh), __builtin_bit_cast(half2v, xvh), acc[b], false);
                            }
                        }
                    }
                }
            }
        }
        if (!has) {                                             // no row, or a row without entries in this bucket
#pragma unroll
            for (int b = 0; b < NB; ++b) acc[b] = 0.f;
        }
        if (nst == 0 && knext < ng) first_steps(knext, nx);    // a group without steps fetched nothing for its successor
        // A row's partial sum goes to its place in the run's partial-sum vector in LDS (rows sit at different lanes in
        // different buckets, so straight from here the 64 lanes would write 64 scattered 4-byte pieces to memory)
        if (split > 1) {
            k_share = kcur;
#pragma unroll
            for (int b = 0; b < NB; ++b) acc_share[b] = acc[b];
        } else if (row != STREAM_SLOT_NONE) {
#pragma unroll
            for (int b = 0; b < NB; ++b) psum[b * a.nl_max + (int)row] = acc[b];
        }
        kcur = knext;
        knext = kafter;
    }
    if (split > 1) {
        // the codebook slice is no longer needed once every wave has left the loop: its LDS holds the shares
        float* share = reinterpret_cast<float*>(lds);
        __syncthreads();
#pragma unroll
        for (int b = 0; b < NB; ++b) share[(wave * NB + b) * 64 + lane] = acc_share[b];
        __syncthreads();
        if (sub == 0 && k_share >= 0) {
            const uint32_t row = slots[(size_t)k_share * 64 + lane] & STREAM_SLOT_NONE;
            if (row != STREAM_SLOT_NONE) {
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    float sum = 0.f;
                    for (int j = 0; j < split; ++j) sum += share[((wave + j) * NB + b) * 64 + lane];
                    psum[b * a.nl_max + (int)row] = sum;
                }
            }
        }
    }
    SQ_TRACE_POINT(2);
    __syncthreads();
    // The run's partial sums leave as whole lines (device-scope stores: written through to memory, so other XCDs'
    // L2s never hold a stale copy).  A partial sum is its own arrival flag: the words of `part` are zero between
    // launches, a sum whose bits are zero travels as STREAM_ZERO_SUM (a NaN pattern no sum can have), and whoever
    // adds a word up puts zero back.  Nobody waits for a store to be acknowledged and there is no arrival counter.
    {
        const int nl = ng * 64;
        uint32_t* pw = reinterpret_cast<uint32_t*>(part) + (size_t)g0 * 64;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (b >= a.nb) break;
            for (int i = tid; i < nl; i += NTH) {
                const uint32_t u = __builtin_bit_cast(uint32_t, psum[b * a.nl_max + i]);
                __hip_atomic_store(pw + b * np + i, u ? u : STREAM_ZERO_SUM, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    SQ_TRACE_POINT(3);
    // Bucket v of the run's NV workgroups finishes share v of the run's (activation row, place) items: it reads the
    // NV partial sums of an item with device-scope loads until none of them is zero, adds them in bucket order, writes
    // y and zeroes the words.  The NV workgroups of a run are neighbours in the grid and workgroups are dispatched in
    // grid order, so a workgroup only ever waits for workgroups that are already running or done; the wait is bounded
    // all the same (an item that gives up is written as NaN).
    const int nl = ng * 64, items = nl * a.nb;
    if constexpr (ORD == 0) {
        if (a.act != nullptr) {
            // SiLU * up on the way out.  The gate and the up piece have the same runs, and a row's partial sums sit at
            // the same place of both pieces' areas, so the 2 NV workgroups of run `wi` of both pieces share the run's
            // rows: each reads the NV sums of the gate row and the NV sums of the up row, finishes both as above, and
            // writes their SiLU product.  (Workgroups of the gate piece then wait for workgroups up to half a launch
            // behind them in the grid: running or done when the launch fits the machine in one round, which the
            // caller's run counts see to; the wait is bounded all the same.)
            const int nf = 2 * P.NV, f = pi * P.NV + v;
            const int e_lo = (int)((int64_t)items * f / nf), e_hi = (int)((int64_t)items * (f + 1) / nf);
            uint32_t* pg = reinterpret_cast<uint32_t*>(a.p[0].part) + (size_t)g0 * 64;
            uint32_t* pu = reinterpret_cast<uint32_t*>(a.p[1].part) + (size_t)g0 * 64;
            const size_t bs = (size_t)NB * np;
            for (int it = e_lo + tid; it < e_hi; it += NTH) {
                const int b = it / nl, i = it - b * nl;
                const uint32_t r = g0 * 64 + i < P.R ? (uint32_t)(g0 * 64 + i) : STREAM_NO_ROW;
                const float rg = h2f(a.p[0].row_scale[r != STREAM_NO_ROW ? r : 0u]), ru = h2f(a.p[1].row_scale[r != STREAM_NO_ROW ? r : 0u]);
                uint32_t* qg = pg + (size_t)b * np + i;
                uint32_t* qu = pu + (size_t)b * np + i;
                uint32_t ug[16], uu[16];
                bool ok = true;
                for (int spin = 0;; ++spin) {
#pragma unroll
                    for (int k = 0; k < 16; ++k) {
                        ug[k] = __hip_atomic_load(qg + (size_t)min(k, P.NV - 1) * bs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        uu[k] = __hip_atomic_load(qu + (size_t)min(k, P.NV - 1) * bs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    ok = true;
#pragma unroll
                    for (int k = 0; k < 16; ++k) ok = ok && ug[k] != 0u && uu[k] != 0u;
                    if (ok || spin >= a.spin_max) break;
                    __builtin_amdgcn_s_sleep(2);
                }
                float sg = 0.f, su = 0.f;
#pragma unroll
                for (int k = 0; k < 16; ++k)
                    if (k < P.NV) {
                        sg += ug[k] == STREAM_ZERO_SUM ? 0.f : __builtin_bit_cast(float, ug[k]);
                        su += uu[k] == STREAM_ZERO_SUM ? 0.f : __builtin_bit_cast(float, uu[k]);
                    }
                for (int k = 0; k < P.NV; ++k) {
                    __hip_atomic_store(qg + (size_t)k * bs, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(qu + (size_t)k * bs, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                if (!ok) {
                    __hip_atomic_store(a.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (a.host_err) __hip_atomic_store(a.host_err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                }
                if (r != STREAM_NO_ROW) {
                    const bool good = ok && err0 == 0u;
                    const uint16_t g16 = round16(good ? sg * rg : __builtin_nanf(""), a.y_dtype);
                    const uint16_t u16 = round16(good ? su * ru : __builtin_nanf(""), a.y_dtype);
                    a.act[(int64_t)b * a.ld_act + r] = silu_mul_one(g16, u16, a.y_dtype);
                }
            }
            return;
        }
    }
    const uint32_t* rows0 = reinterpret_cast<const uint32_t*>(P.stream + P.off_rows) + (size_t)g0 * 64;
    const int i_lo = (int)((int64_t)items * v / P.NV), i_hi = (int)((int64_t)items * (v + 1) / P.NV);
    uint32_t* pp = reinterpret_cast<uint32_t*>(P.part) + (size_t)g0 * 64;
    const size_t ysz = a.y_dtype == SQ_F32 ? 4 : 2;
    for (int it = i_lo + tid; it < i_hi; it += NTH) {
        const int b = it / nl, i = it - b * nl;
        const uint32_t r = perms ? rows0[i] : (g0 * 64 + i < P.R ? (uint32_t)(g0 * 64 + i) : STREAM_NO_ROW);
        const float rs = h2f(P.row_scale[r != STREAM_NO_ROW ? r : 0u]);
        uint32_t* q = pp + (size_t)b * np + i;
        const size_t bs = (size_t)NB * np;                      // words from one bucket's partial sums to the next
        float sum = 0.f;
        bool ok = true;
        if (P.NV <= 16) {
            uint32_t u[16];
            for (int spin = 0;; ++spin) {
                // (unconditional loads from clamped indices: all of them are in flight together)
#pragma unroll
                for (int k = 0; k < 16; ++k) u[k] = __hip_atomic_load(q + (size_t)min(k, P.NV - 1) * bs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ok = true;
#pragma unroll
                for (int k = 0; k < 16; ++k) ok = ok && u[k] != 0u;
                if (ok || spin >= a.spin_max) break;
                __builtin_amdgcn_s_sleep(2);
            }
#pragma unroll
            for (int k = 0; k < 16; ++k)
                if (k < P.NV) sum += u[k] == STREAM_ZERO_SUM ? 0.f : __builtin_bit_cast(float, u[k]);
        } else {
            for (int v0 = 0; v0 < P.NV; v0 += 32) {
                uint32_t u[32];
                for (int spin = 0;; ++spin) {
#pragma unroll
                    for (int k = 0; k < 32; ++k) u[k] = __hip_atomic_load(q + (size_t)min(v0 + k, P.NV - 1) * bs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    bool all = true;
#pragma unroll
                    for (int k = 0; k < 32; ++k) all = all && u[k] != 0u;
                    if (all) break;
                    if (spin >= a.spin_max) { ok = false; break; }
                    __builtin_amdgcn_s_sleep(2);
                }
#pragma unroll
                for (int k = 0; k < 32; ++k)
                    if (v0 + k < P.NV) sum += u[k] == STREAM_ZERO_SUM ? 0.f : __builtin_bit_cast(float, u[k]);
            }
        }
        for (int k = 0; k < P.NV; ++k) __hip_atomic_store(q + (size_t)k * bs, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (!ok) {
            // gave up: the missing sums may still arrive and stay in the header, so the workspace is marked unusable
            __hip_atomic_store(a.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (a.host_err) __hip_atomic_store(a.host_err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        if (r != STREAM_NO_ROW)
            store_y((char*)a.y + (size_t)b * a.ldy * ysz, a.y_dtype, (int64_t)P.y_off + r, ok && err0 == 0u ? sum * rs : __builtin_nanf(""));
    }
    SQ_TRACE_POINT(6);
}

// LDS bytes of a launch: slice, NB parts of x, NB partial-sum vectors of the longest run, flags, block sums
static size_t stream_smem(int nb_t, int xs, int nl_max, int xcopies = 1, int xtmp = 0) {
    return (size_t)STREAM_TAB + (size_t)xcopies * nb_t * xs + (size_t)nb_t * nl_max * 4 + 16 + 64 + (size_t)nb_t * xtmp;
}

template <int NB, int NX, int PRO, int ORD, int NAR>
static int stream_launch_as(const StreamArgs& a, int grid, hipStream_t s) {
    // (the attribute is a property of the function, the same on every device; setting it twice from two threads is harmless)
    static std::atomic<bool> raised{false};
    if (!raised.load(std::memory_order_acquire)) {
        (void)hipFuncSetAttribute((const void*)stream_kernel<NB, NX, PRO, ORD, NAR>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        (void)hipGetLastError();
        raised.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL((stream_kernel<NB, NX, PRO, ORD, NAR>), dim3((unsigned)grid), dim3(STREAM_NW * 64), stream_smem(NB, a.xs, a.nl_max, a.xcopies, a.xtmp_own ? a.xtmp : 0), s, a);
    return check_launch("sq_linear_small(stream)");
}
// (a.orders: some piece of the launch has column orders; a.narrow: the pieces' entry format)
template <int NB, int NX, int PRO = 0>
static int stream_launch(const StreamArgs& a, int grid, hipStream_t s) {
    if (PRO != 0) {
        if (a.orders) return fail(SQ_EUNSUPPORTED, "sq_linear_small_from: no fused kernel for pieces with column orders");
        return a.narrow ? stream_launch_as<NB, NX, PRO, 0, 1>(a, grid, s) : stream_launch_as<NB, NX, PRO, 0, 0>(a, grid, s);
    }
    if (a.narrow) return a.orders ? stream_launch_as<NB, NX, 0, 1, 1>(a, grid, s) : stream_launch_as<NB, NX, 0, 0, 1>(a, grid, s);
    return a.orders ? stream_launch_as<NB, NX, 0, 1, 0>(a, grid, s) : stream_launch_as<NB, NX, 0, 0, 0>(a, grid, s);
}

// ---- dense rows from the tag stream alone (a matrix held in one copy: sq_matrix.tags == NULL).  One wave per (bucket,
// group): lane = row, as in the product; every real entry writes its chunk of 8 weights, so over all buckets each
// (row, chunk) is written exactly once.  Same arithmetic as dequant_kernel: f32(codeword) * f32(row scale), one rounding.
struct StreamDeqArgs {
    const unsigned char* stream;
    const uint16_t* table;
    const uint16_t* row_scale;
    const uint8_t* row_mask;
    const int32_t* perms;
    void* out;
    int64_t ld_out;
    int R, C, NS, NV, PC, NG, fs, r0, r1, raw, vec;
    uint32_t off_slots, off_rows, off_steps;
};

template <int DT, int NAR>
__global__ __launch_bounds__(256) void stream_dequant_kernel(StreamDeqArgs a) {
    typedef typename store_as<DT>::type T;
    typedef StreamF<NAR> F;
    constexpr int STREAM_PF = F::PF;
    const int lane = threadIdx.x & 63;
    const int w = (int)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (w >= a.NV * a.NG) return;
    const int v = w / a.NG, s = v % a.NS, kp = v / a.NS;
    const u32x4 hw = reinterpret_cast<const u32x4*>(a.stream)[w];             // {rest, nst, unit0, split | g0 << 8}
    const int nst = (int)hw.y, split = (int)(hw.w & 0xFFu);
    const uint32_t slot = reinterpret_cast<const uint16_t*>(a.stream + a.off_slots)[(size_t)w * 64 + lane];
    uint32_t row = STREAM_NO_ROW;
    if ((slot & STREAM_SLOT_NONE) != STREAM_SLOT_NONE) {
        const uint32_t place = (slot & STREAM_SLOT_NONE) + (hw.w >> 8) * 64u;
        row = a.perms ? reinterpret_cast<const uint32_t*>(a.stream + a.off_rows)[place] : place;
    }
    const bool mine = row != STREAM_NO_ROW && (int)row >= a.r0 && (int)row < a.r1 && (slot & STREAM_SLOT_HAS) != 0u;
    if (__ballot(mine) == 0) return;                             // (wave-uniform) none of this group's rows is wanted
    const float sc = (mine && !a.raw) ? h2f(a.row_scale[row]) : 1.f;
    const int32_t* pm = (mine && a.perms) ? a.perms + (size_t)(a.row_mask ? a.row_mask[row] : 0) * a.C : nullptr;
    T* orow = reinterpret_cast<T*>(a.out) + (mine ? (int64_t)((int)row - a.r0) * a.ld_out : 0);
    const unsigned char* rec = a.stream + a.off_steps + lane * F::LB;
    int j = 0, s0 = 0, s1 = nst / split;                          // the share step t belongs to, its first and end step
    for (int t = 0; t < nst; ++t) {
        while (t >= s1) { ++j; s0 = s1; s1 = nst * (j + 1) / split; }
        const size_t at = t - s0 < STREAM_PF ? ((size_t)(hw.z + (uint32_t)j) * a.NV + v) * a.fs + (size_t)(t - s0)
                                             : (size_t)hw.x + (size_t)t - (size_t)STREAM_PF * (j + 1);
        uint32_t e[F::EPS];
        F::entries(*reinterpret_cast<const typename F::vec*>(rec + at * F::SB), e);
#pragma unroll
        for (int j = 0; j < F::EPS; ++j) {
            // (padding entries name one of the zero chunks behind the part's own)
            const int cj = (int)((e[j] >> STREAM_SLICE_BITS) & F::CMASK);
            if (!mine || cj >= a.PC) continue;
            const uint32_t tag = (e[j] & 0xFFFu) + ((uint32_t)s << STREAM_SLICE_BITS);
            const int c0 = (cj + kp * a.PC) * 8;
            const u32x4 cw = *reinterpret_cast<const u32x4*>(a.table + (size_t)tag * 8);
            T o[8];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t pair = cw[k];
                o[2 * k] = store_as<DT>::cvt(h2f((uint16_t)(pair & 0xFFFFu)) * sc);
                o[2 * k + 1] = store_as<DT>::cvt(h2f((uint16_t)(pair >> 16)) * sc);
            }
            if (pm) {
#pragma unroll
                for (int k = 0; k < 8; ++k) orow[pm[c0 + k]] = o[k];
            } else if (a.vec) {
                constexpr int PER = 16 / (int)sizeof(T);         // elements per 16-byte store
#pragma unroll
                for (int q = 0; q < 8 / PER; ++q) {
                    u32x4 pk;
                    __builtin_memcpy(&pk, o + q * PER, 16);
                    *reinterpret_cast<u32x4*>(orow + c0 + q * PER) = pk;
                }
            } else {
#pragma unroll
                for (int k = 0; k < 8; ++k) orow[c0 + k] = o[k];
            }
        }
    }
}

int launch_stream_dequant(const sq_matrix& m, void* out, int out_dtype, int64_t ld_out, int r0, int r1, hipStream_t s, bool raw) {
    if (!stream_shape(m)) return fail(SQ_EINVAL, "sq_dequant: a matrix without tags needs its tag stream");
    const StreamGeom g = stream_geom_of(m);
    StreamDeqArgs a;
    a.stream = (const unsigned char*)m.stream;
    a.table = g.off_table ? (const uint16_t*)((const unsigned char*)m.stream + g.off_table) : m.table; a.row_scale = m.row_scale; a.row_mask = m.row_mask; a.perms = m.perms;
    a.out = out; a.ld_out = ld_out; a.R = m.R; a.C = m.C; a.NS = g.NS; a.NV = g.NV; a.PC = g.PC; a.NG = g.NG; a.fs = g.fs; a.r0 = r0; a.r1 = r1;
    a.raw = raw ? 1 : 0;
    a.off_slots = (uint32_t)g.off_slots; a.off_rows = (uint32_t)g.off_rows; a.off_steps = (uint32_t)g.off_steps;
    const size_t es = out_dtype == SQ_F32 ? 4 : 2;
    a.vec = ((uintptr_t)out & 15) == 0 && (ld_out * es) % 16 == 0;
    const unsigned grid = (unsigned)(((int64_t)g.NV * g.NG + 3) / 4);
#define SQ_DEQ(DT) do { if (g.fmt.narrow) hipLaunchKernelGGL((stream_dequant_kernel<DT, 1>), dim3(grid), dim3(256), 0, s, a); \
                        else hipLaunchKernelGGL((stream_dequant_kernel<DT, 0>), dim3(grid), dim3(256), 0, s, a); } while (0)
    switch (out_dtype) {
        case SQ_F32: SQ_DEQ(SQ_F32); break;
        case SQ_F16: SQ_DEQ(SQ_F16); break;
        case SQ_BF16: SQ_DEQ(SQ_BF16); break;
        default: return fail(SQ_EINVAL, "sq_dequant: out_dtype %d", out_dtype);
    }
#undef SQ_DEQ
    return check_launch("sq_dequant(stream)");
}

bool stream_shape(const sq_matrix& m) {
    return m.stream && stream_runs_of(m) > 0 && m.stream_groups > 0 && stream_format_ok(m.R, m.C, m.d, m.bits, m.G) &&
           !(m.G > 1 && stream_balanced_of(m)) &&
           (m.M <= 1 || m.perms) && (((uintptr_t)m.table | (uintptr_t)m.stream | (uintptr_t)m.perms) & 15) == 0 &&
           stream_part_bytes(m, 1) <= SQ_WS_SUMS;
}

// ---- the error word's host-visible copy and the spin limit
static std::atomic<int> g_stream_spin{STREAM_SPIN_MAX};
static std::atomic<uint32_t*> g_host_flag[64];          // per device: pinned host word
static std::atomic<uint32_t*> g_host_flag_dev[64];      // its address as the device sees it

void stream_set_spin(int polls) { g_stream_spin.store(polls < 0 ? STREAM_SPIN_MAX : polls, std::memory_order_relaxed); }

static int current_device() {
    int dev = 0;
    return hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 ? dev : -1;
}

uint32_t* stream_host_flag(hipStream_t s, bool may_allocate) {
    const int dev = current_device();
    if (dev < 0) return nullptr;
    uint32_t* d = g_host_flag_dev[dev].load(std::memory_order_acquire);
    if (d || !may_allocate) return d;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &st) != hipSuccess || st != hipStreamCaptureStatusNone) { (void)hipGetLastError(); return nullptr; }
    static std::mutex mu;
    std::lock_guard<std::mutex> lock(mu);
    d = g_host_flag_dev[dev].load(std::memory_order_acquire);
    if (d) return d;
    void* h = nullptr;
    void* hd = nullptr;
    if (hipHostMalloc(&h, 64, hipHostMallocMapped) != hipSuccess || !h || hipHostGetDevicePointer(&hd, h, 0) != hipSuccess || !hd) {
        (void)hipGetLastError();
        if (h) (void)hipHostFree(h);
        return nullptr;
    }
    *reinterpret_cast<volatile uint32_t*>(h) = 0u;
    g_host_flag[dev].store(reinterpret_cast<uint32_t*>(h), std::memory_order_release);
    g_host_flag_dev[dev].store(reinterpret_cast<uint32_t*>(hd), std::memory_order_release);
    return reinterpret_cast<uint32_t*>(hd);
}

bool stream_host_flag_set() {
    const int dev = current_device();
    const uint32_t* h = dev < 0 ? nullptr : g_host_flag[dev].load(std::memory_order_acquire);
    return h && *reinterpret_cast<const volatile uint32_t*>(h) != 0u;
}

void stream_host_flag_clear() {
    const int dev = current_device();
    uint32_t* h = dev < 0 ? nullptr : g_host_flag[dev].load(std::memory_order_acquire);
    if (h) *reinterpret_cast<volatile uint32_t*>(h) = 0u;
}

// rows of one pass: 1, 2, 4 or 8
int stream_pass_rows(int B) { return B > 4 ? 8 : B > 2 ? 4 : B > 1 ? 2 : 1; }

size_t stream_part_bytes(const sq_matrix& m, int rows) {
    const StreamGeom g = stream_geom_of(m);
    return (((size_t)g.NV * rows * g.NG * 64 * 4) + 255) & ~(size_t)255;
}

int stream_group_len(const sq_matrix* mats, int n) {
    size_t tot = 0;
    int k = 0;
    for (; k < n; ++k) {
        tot += stream_part_bytes(mats[k], 1);
        if (tot > SQ_WS_SUMS) break;
    }
    return k > 0 ? k : 1;
}

// Pieces [0, cnt) (same C), B activation rows in passes of up to 8 (fewer when the parts of x and the runs' partial
// sums of that many rows do not fit LDS beside the slice, or the pieces' partial sums of that many rows the workspace
// header): one launch per pass.  `sums` is the workspace header; every pass uses it from its start (a pass leaves it zeroed).
int launch_stream_group(const sq_matrix* mats, int cnt, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                        int64_t ldy, int B, char* sums, hipStream_t s, const sq_producer* from, void* act, int64_t ld_act) {
    StreamArgs a;
    a.act = (uint16_t*)act;
    a.ld_act = ld_act;
    if (act) {
        // (what stream_fuses_silu() promises; checked again where the kernel depends on it)
        if (cnt != 2 || mats[0].perms || mats[1].perms || mats[0].R != mats[1].R || stream_runs_of(mats[0]) != stream_runs_of(mats[1]) ||
            mats[0].stream_groups != mats[1].stream_groups || y_dtype == SQ_F32 || stream_geom_of(mats[0]).NV > 16)
            return fail(SQ_EINVAL, "sq_linear_small_silu: the two pieces must be a gate and an up projection of one shape");
    }
    a.h_in = nullptr; a.h_out = nullptr; a.add = a.w = nullptr; a.x_out = nullptr; a.eps = 0.f;
    if (from) {
        a.h_in = from->h_in; a.h_out = from->h_out; a.add = (const uint16_t*)from->add;
        a.w = (const uint16_t*)from->w; a.x_out = (uint16_t*)from->x_out; a.eps = from->eps;
    }
    a.err = reinterpret_cast<uint32_t*>(sums + SQ_WS_ERR_OFF);
    a.host_err = stream_host_flag(s, false);
    a.spin_max = g_stream_spin.load(std::memory_order_relaxed);
    a.n = cnt;
    a.ldx = ldx;
    a.ldy = ldy;
    a.x_dtype = x_dtype;
    a.y_dtype = y_dtype;
    int rows = from ? 1 : stream_pass_rows(B);
    for (;; rows >>= 1) {
        size_t tot = 0;
        for (int k = 0; k < cnt; ++k) tot += stream_part_bytes(mats[k], rows);
        if (tot <= SQ_WS_SUMS) break;
        if (rows == 1) return fail(SQ_EUNSUPPORTED, "sq_linear_small: the partial sums of these pieces (%zu bytes) do not fit the workspace header", tot);
    }
    int wg = 0, pc = 0, nl_max = 64, xcopies = 1, xtmp = 0;
    a.orders = 0;
    bool one_part = true;                                       // every piece with column orders has one column part
    size_t sums_off = 0;
    for (int k = 0; k < cnt; ++k) {
        const sq_matrix& m = mats[k];
        const int runs = stream_runs_of(m), run_max = stream_run_max_of(m);
        const StreamGeom g = stream_geom_of(m);
        if (m.stream_groups < (m.R + 63) / 64 || runs > m.stream_groups || runs < 1 || run_max < 1 || run_max > STREAM_RUN_MAX)
            return fail(SQ_EINVAL, "sq_linear_small: stream_runs 0x%x / stream_groups %d do not fit %d rows", m.stream_runs, m.stream_groups, m.R);
        // Without column orders the kernel cuts the groups into runs of ceil(groups / runs) itself: a run count that
        // leaves the last run empty, or whose runs are longer than the buffer says, is not one the builder made.
        const int gr = (g.NG + runs - 1) / runs;
        if (!m.perms && ((runs - 1) * gr >= g.NG || gr != run_max))
            return fail(SQ_EINVAL, "sq_linear_small: stream_runs 0x%x does not cut %d groups the way the builder does", m.stream_runs, m.stream_groups);
        StreamPiece& P = a.p[k];
        P.stream = (const unsigned char*)m.stream;
        P.table = g.off_table ? (const uint16_t*)((const unsigned char*)m.stream + g.off_table) : m.table;
        P.row_scale = m.row_scale;
        P.part = (float*)(sums + sums_off);
        sums_off += stream_part_bytes(m, rows);
        P.perms = m.perms;
        P.R = m.R; P.C = m.C; P.U = g.U; P.NS = g.NS; P.NV = g.NV; P.PC = g.PC; P.NG = g.NG; P.y_off = m.y_off;
        P.fs = g.fs;
        P.off_slots = (uint32_t)g.off_slots; P.off_runs = (uint32_t)g.off_runs; P.off_rows = (uint32_t)g.off_rows;
        P.off_steps = (uint32_t)g.off_steps;
        const int nwg = g.runs;
        P.wg_begin = wg;
        P.nwg = nwg;
        wg += g.NV * nwg;
        pc = g.PC;                                               // (pieces of one launch share C)
        nl_max = std::max(nl_max, run_max * 64);
        if (m.perms) {
            a.orders = 1;
            xcopies = std::max(xcopies, stream_run_orders_of(m));
            xtmp = std::max(xtmp, (m.C * 2 + 15) & ~15);
            one_part = one_part && g.U == g.PC;
        }
    }
    for (int k = cnt; k < GEMV_MAX_PIECES_STREAM; ++k) a.p[k] = a.p[0];
    a.xs = stream_xs(pc);
    a.narrow = stream_fmt(pc).narrow;
    a.nl_max = nl_max;
    a.xcopies = xcopies;
    a.xtmp = a.xtmp_own = 0;
    if (from || !one_part) xtmp = 0;                            // (produced rows and rows of several parts: gathered from memory)
    if (stream_smem(1, a.xs, a.nl_max, xcopies) > 160 * 1024 || pc * xcopies > 4 * STREAM_NW * 64)
        return fail(SQ_EUNSUPPORTED, "sq_linear_small: %d copies of a row part of %d chunks do not fit LDS", xcopies, pc);
    const bool nx4 = pc * xcopies > STREAM_NW * 64;             // chunks of x (over all its copies) per thread: 1 or 4
    if (from) {
        if (B != 1) return fail(SQ_EINVAL, "sq_linear_small_from: fused producers take one activation row");
        a.x = (const uint16_t*)x; a.y = y; a.nb = 1;
        if (from->mode != SQ_FROM_ADDNORM) return fail(SQ_EINVAL, "sq_linear_small_from: only add + norm is produced inside the kernel");
        return nx4 ? stream_launch<1, 4, 1>(a, wg, s) : stream_launch<1, 1, 1>(a, wg, s);
    }
    while (rows > 1 && stream_smem(rows, a.xs, a.nl_max, xcopies) > 160 * 1024) rows >>= 1;
    // Column orders are applied from copies of the rows in LDS: in LDS of their own where that is left, else where
    // the slice lands afterwards (that part of the slice is then copied a round trip later), if they fit there.
    a.xtmp_own = xtmp > 0 && stream_smem(rows, a.xs, a.nl_max, xcopies, xtmp) <= 160 * 1024;
    a.xtmp = a.xtmp_own || rows * xtmp <= STREAM_TAB ? xtmp : 0;
    const size_t ysz = y_dtype == SQ_F32 ? 4 : 2;
    for (int b0 = 0; b0 < B; b0 += rows) {
        a.x = (const uint16_t*)((const char*)x + (size_t)b0 * ldx * 2);
        a.y = y ? (char*)y + (size_t)b0 * ldy * ysz : nullptr;
        a.act = act ? (uint16_t*)act + (size_t)b0 * ld_act : nullptr;
        a.nb = std::min(rows, B - b0);
        int rc;
        switch (rows) {
            case 1: rc = nx4 ? stream_launch<1, 4>(a, wg, s) : stream_launch<1, 1>(a, wg, s); break;
            case 2: rc = nx4 ? stream_launch<2, 4>(a, wg, s) : stream_launch<2, 1>(a, wg, s); break;
            case 4: rc = nx4 ? stream_launch<4, 4>(a, wg, s) : stream_launch<4, 1>(a, wg, s); break;
            default: rc = nx4 ? fail(SQ_ELAUNCH, "sq_linear_small: 8 rows of more than 1024 chunks cannot fit LDS") : stream_launch<8, 1>(a, wg, s); break;
        }
        if (rc) return rc;
    }
    return SQ_OK;
}

}  // namespace sq
