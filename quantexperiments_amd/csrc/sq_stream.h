// Geometry of the bucketed tag stream shared by its host-side builder, the launcher and the kernel.
#pragma once
#include <functional>
#include "sq_common.h"

namespace sq {

constexpr int STREAM_SLICE_BITS = 12;        // 4096 codewords of 16 bytes per LDS slice
constexpr int STREAM_PART_MAX = 640;         // most chunks in one column part (10 bits of an entry are enough)
constexpr int STREAM_ZERO_CHUNK = STREAM_PART_MAX;   // chunk index of padding entries: a chunk of x kept at zero
constexpr int STREAM_ROW_BITS = 19;          // slot = row | count << 19
constexpr uint32_t STREAM_NO_ROW = (1u << STREAM_ROW_BITS) - 1u;
constexpr int GEMV_MAX_PIECES_STREAM = 4;

constexpr int STREAM_DEFAULT_WGS = 512;      // workgroups a matrix launched alone should make (2 per CU on 256 CUs)

struct StreamGeom {
    int U, NS, KP, PC, NV, NG;               // chunks per row, slices, column parts, chunks per part, buckets, groups
    int runs;
    size_t off_slots, off_runs, off_rows, off_steps;   // byte offsets inside the stream buffer
    uint64_t total_steps;                    // filled by the builder only
};

StreamGeom stream_geom(int C, int d, int bits, int groups, int runs);
bool stream_format_ok(int R, int C, int d, int bits);
size_t stream_bytes_host(const uint32_t* tags, int R, int W, int C, int d, int bits, const uint8_t* row_mask, int runs);
int stream_build_host(const uint32_t* tags, int R, int W, int C, int d, int bits, const uint8_t* row_mask, int runs,
                      unsigned char* out, size_t bytes, int* runs_out, int* groups_out);
bool stream_shape(const sq_matrix& m);
size_t stream_part_bytes(const sq_matrix& m, int B);
int launch_stream_group(const sq_matrix* mats, int cnt, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                        int64_t ldy, int nb, int B, char* ws, size_t& ws_off, unsigned* counters, int& counters_used,
                        hipStream_t s, const sq_producer* from = nullptr);

}  // namespace sq
