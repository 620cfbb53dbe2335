// Geometry of the bucketed tag stream shared by its host-side builder, the launcher and the kernel.
#pragma once
#include <functional>
#include "sq_common.h"

namespace sq {

constexpr int STREAM_SLICE_BITS = 12;        // 4096 codewords of 16 bytes per LDS slice
constexpr int STREAM_PART_MAX = 4064;        // most chunks in one column part: its chunks and the 16 zero chunks that padding
                                             // entries multiply with (chunks PC .. PC + 15 of the part) fit 12 bits of an entry
constexpr int STREAM_RUN_MAX = 96;           // most groups of 64 rows in one run (a run's partial sums are staged in LDS)
constexpr int STREAM_ROW_BITS = 19;          // places (indices into the row list) stay below 2^19
constexpr uint32_t STREAM_NO_ROW = (1u << STREAM_ROW_BITS) - 1u;
// Slot of a lane (16 bits per lane, group and bucket): the lane's row as its place counted from the run's first place
// (a run has at most STREAM_RUN_MAX * 64 = 6144 places), STREAM_SLOT_NONE for a lane without a row, and
// STREAM_SLOT_HAS when the row has entries in the bucket (a lane without any walks a neighbour's entries and its sum is
// dropped).
constexpr uint32_t STREAM_SLOT_NONE = 0x1FFFu;
constexpr uint32_t STREAM_SLOT_HAS = 0x2000u;
// Entry formats.  Wide: 24 bits (12-bit tag within the slice, 12-bit chunk within the column part), four per lane and
// step in 12 bytes, steps of 768 bytes.  Narrow, for column parts of at most STREAM_NARROW_MAX chunks (9 bits name the
// part's chunks and the 16 zero chunks behind them): 21 bits (12 + 9), three per lane and step in 8 bytes (entry i at
// bits 21 i of the lane's 64), steps of 512 bytes.  Either way a prefetch batch is 12 entries per lane.
constexpr int STREAM_NARROW_MAX = 496;
struct StreamFmt { int narrow, eps, lane_bytes, step_bytes, pf, chunk_bits; };
__host__ __device__ inline StreamFmt stream_fmt(int PC) {
    return PC <= STREAM_NARROW_MAX ? StreamFmt{1, 3, 8, 512, 4, 9} : StreamFmt{0, 4, 12, 768, 3, 12};
}
constexpr int GEMV_MAX_PIECES_STREAM = 4;
constexpr int STREAM_RUN_ORDERS = 8;         // most column orders whose rows may share a run (one gathered copy of x in LDS each)

constexpr int STREAM_DEFAULT_WGS = 256;      // workgroups a matrix launched alone should make (one per CU on 256 CUs)
constexpr int STREAM_NW = 16;                // waves per workgroup of the kernel: one workgroup per CU
// Steps the kernel fetches ahead = StreamFmt.pf (12 entries per lane; 2 to 4 wide steps measure alike, 6 and 8 slower);
// the first of every unit's steps are kept in the first-steps region.

// A unit is what one wave walks without a break: a group of a run, or, in a run of at most STREAM_NW / 2 groups, one of
// the STREAM_NW / groups contiguous shares of a group's steps (share j of `split`: steps [nst j / split, nst (j + 1) / split)).
__host__ __device__ inline int stream_split_of(int ng) { return ng * 2 <= STREAM_NW ? STREAM_NW / ng : 1; }

// Where the steps are (all positions in steps from off_steps; PF = StreamFmt.pf).  The first FS steps of every unit sit
// in a region of their own, at a place that follows from the unit's index alone: ((unit * NV + bucket) * FS), so a
// wave can ask for them before it has read anything else of the buffer; a launch then starts with one round trip to
// memory instead of two (offsets, then steps).  FS is PF, or, in a matrix none of whose units has that many steps (short
// shares of small matrices), the longest unit's step count.  The remaining steps of a group follow each other in the
// rest region, share after share.  Per (bucket, group) the buffer holds four words: {rest, nst, unit0, split | g0 << 8}
// = the place of the group's first remaining step, its step count, the index of its first unit, its share count and the
// first group of its run; when every share has at least PF steps (nst / split >= PF), step t of share j (t counted
// within the group) is at rest + t - PF (j + 1) once it is past the share's first PF; otherwise the first-steps region
// holds the whole group.

struct StreamGeom {
    int U, NS, KP, PC, NV, NG;               // chunks per row, slices, column parts, chunks per part, buckets, groups
    int runs;
    int fs;                                  // steps per unit in the first-steps region (1 .. fmt.pf)
    StreamFmt fmt;
    size_t off_slots, off_runs, off_rows, off_steps;   // byte offsets inside the stream buffer
    size_t off_table, off_unmap;             // balanced streams: the relabelled codebook and uint16 new id -> file id (else 0)
    uint64_t total_steps;                    // filled by the builder only
};

// Several codebooks per matrix (G, a power of two; row_book[r] names the row's): the G codebooks lie behind each other in
// the table, so a row's tags become labels of that one long codebook, book << bits | tag, and everything below (slices,
// buckets, the kernels) sees a matrix with one codebook of G << bits codewords: `label_bits` = bits + log2 G.  The
// workgroups of a slice then find entries only in the rows of that slice's codebook.
constexpr int STREAM_SLICES_MAX = 64;        // most slices of one matrix (4 MiB of codebooks): the workgroups of a run wait for
                                             // each other and must be resident together
inline int stream_label_bits(int bits, int G) {
    int lb = bits;
    while (G > 1) { G >>= 1; ++lb; }
    return lb;
}
StreamGeom stream_geom(int C, int d, int label_bits, int groups, int runs, bool balanced = false, int fs = 0);
bool stream_format_ok(int R, int C, int d, int bits, int G = 1);
// table: the matrix' codebook (fp16 [2^bits, d], host memory; one codebook only) or NULL.  With it the codewords are
// relabelled so that every slice of 4096 carries the same share of the tags whatever their distribution, and the buffer
// holds the relabelled copy of the codebook that the kernels then read their slices from.
size_t stream_bytes_host(const uint32_t* tags, int R, int W, int C, int d, int bits, const uint8_t* row_mask, int runs,
                         const uint16_t* table = nullptr, int G = 1, const uint8_t* row_book = nullptr);
int stream_build_host(const uint32_t* tags, int R, int W, int C, int d, int bits, const uint8_t* row_mask, int runs,
                      unsigned char* out, size_t bytes, int* runs_out, int* groups_out, const uint16_t* table = nullptr,
                      int G = 1, const uint8_t* row_book = nullptr);
// remap_out[book << bits | file label] = new label within the book (G << bits entries): the relabelling a balanced stream
// applies, by itself; every codebook is balanced over its own slices (one of at most 4096 codewords keeps its labels)
void stream_balance_host(const uint32_t* tags, int R, int W, int C, int d, int bits, uint16_t* remap_out, int G = 1,
                         const uint8_t* row_book = nullptr);
// sq_matrix.stream_runs is sq_stream_build's runs_out: the run count in the low 16 bits, the groups of the longest run
// in the next 8, the most column orders in one run (less one) in bits 24-26, the steps per unit of the first-steps region
// (less one) in bits 27-28, bit 30 = the stream carries a relabelled codebook
constexpr int STREAM_BALANCED = 1 << 30;
inline int stream_fs_of(const sq_matrix& m) { return (int)(((uint32_t)m.stream_runs >> 27) & 3u) + 1; }
inline int stream_runs_of(const sq_matrix& m) { return m.stream_runs & 0xFFFF; }
inline int stream_run_max_of(const sq_matrix& m) { return (int)(((uint32_t)m.stream_runs >> 16) & 0xFFu); }
inline int stream_run_orders_of(const sq_matrix& m) { return (int)(((uint32_t)m.stream_runs >> 24) & 7u) + 1; }
inline bool stream_balanced_of(const sq_matrix& m) { return (m.stream_runs & STREAM_BALANCED) != 0; }
inline StreamGeom stream_geom_of(const sq_matrix& m) {
    return stream_geom(m.C, m.d, stream_label_bits(m.bits, m.G), m.stream_groups, stream_runs_of(m), stream_balanced_of(m), stream_fs_of(m));
}
bool stream_shape(const sq_matrix& m);
size_t stream_part_bytes(const sq_matrix& m, int rows);   // partial sums of one pass of `rows` activation rows
// dense rows [r0, r1) of a matrix that is held as its tag stream only (sq_matrix.tags == NULL)
int launch_stream_dequant(const sq_matrix& m, void* out, int out_dtype, int64_t ld_out, int r0, int r1, hipStream_t s, bool raw);
// act != NULL (two pieces of one shape, gate and up, no column orders, a 16-bit y_dtype): y is not written, act[b * ld_act + r]
// = silu(Y[b, r]) * Y[b, R + r] is
int launch_stream_group(const sq_matrix* mats, int cnt, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                        int64_t ldy, int B, char* sums, hipStream_t s, const sq_producer* from = nullptr, void* act = nullptr,
                        int64_t ld_act = 0);
// pieces [0, n) a single launch can take: their partial sums of one activation row fit the workspace header together
int stream_group_len(const sq_matrix* mats, int n);
// activation rows the kernel takes per pass for B of them (1, 2, 4 or 8)
int stream_pass_rows(int B);
// Polls of an item's partial sums before a workgroup gives up (sq_stream_spin_limit); and this device's host-visible
// copy of the error word, which a workgroup that gives up also sets so that the next call can refuse without a
// synchronisation: its device address (NULL when there is none and `may_allocate` is false, or under stream capture),
// whether it is set, and its clearing.
void stream_set_spin(int polls);
uint32_t* stream_host_flag(hipStream_t s, bool may_allocate);
bool stream_host_flag_set();
void stream_host_flag_clear();

}  // namespace sq
