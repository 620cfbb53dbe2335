// Shared device helpers for the gfx950 codebook-linear kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/sqhip.h"

namespace sq {

typedef _Float16 half_t;
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int WAVE = 64;

__device__ __forceinline__ float h2f(uint16_t b) { return (float)__builtin_bit_cast(half_t, b); }
__device__ __forceinline__ float bf2f(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }

// fp32 -> bf16 bits, round to nearest even, NaN stays NaN.
__device__ __forceinline__ uint16_t f2bf(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
// fp32 -> fp16 bits, round to nearest even.  The empty asm hides where f came from: a multiply feeding this conversion
// is otherwise folded into v_fma_mixlo_f16, which rounds the exact product to fp16 once, while the same expression
// elsewhere in a kernel stays v_mul_f32 + v_cvt_f16_f32 (two roundings, the reference's arithmetic) and differs in
// the last bit of about one value in 2000.
__device__ __forceinline__ uint16_t f2h(float f) {
    asm("" : "+v"(f));
    return __builtin_bit_cast(uint16_t, (half_t)f);
}

// bf16 bits -> fp16 value (through fp32; exact whenever the value is an fp16 normal,
// rounds to nearest even in the fp16 subnormal range, +-inf beyond 65504).
__device__ __forceinline__ half_t bf2h(uint16_t b) { return (half_t)bf2f(b); }

// two packed bf16 (one dword) -> two packed fp16
__device__ __forceinline__ uint32_t bf2h_x2(uint32_t v) {
    half2v h;
    h.x = (half_t)__builtin_bit_cast(float, v << 16);
    h.y = (half_t)__builtin_bit_cast(float, v & 0xFFFF0000u);
    return __builtin_bit_cast(uint32_t, h);
}

// 16-bit activations of a run-time dtype (SQ_F16 / SQ_BF16)
__device__ __forceinline__ float load16(const void* p, int dtype, int64_t i) {
    const uint16_t b = reinterpret_cast<const uint16_t*>(p)[i];
    return dtype == SQ_BF16 ? bf2f(b) : h2f(b);
}
__device__ __forceinline__ uint16_t round16(float v, int dtype) { return dtype == SQ_BF16 ? f2bf(v) : f2h(v); }

// silu(g) * u with the reference's rounding points (shapequant/kernels/decode_e2e.py:125-136): SiLU in fp32 rounded
// to the model dtype, then the product rounded to the model dtype.  One definition, because the stand-alone kernel
// and the products that compute their own input must agree bit for bit.
__device__ __forceinline__ uint16_t silu_mul_one(uint16_t g, uint16_t u, int dtype) {
    if (dtype == SQ_BF16) {
        const float a = bf2f(g);
        return f2bf(bf2f(f2bf(a / (1.f + __expf(-a)))) * bf2f(u));
    }
    const float a = h2f(g);
    const half_t s = (half_t)(a / (1.f + __expf(-a)));
    return __builtin_bit_cast(uint16_t, (half_t)(s * __builtin_bit_cast(half_t, u)));
}

template <int DT> struct store_as;
template <> struct store_as<SQ_F32> { typedef float type; static __device__ __forceinline__ float cvt(float f) { return f; } };
template <> struct store_as<SQ_F16> { typedef uint16_t type; static __device__ __forceinline__ uint16_t cvt(float f) { return f2h(f); } };
template <> struct store_as<SQ_BF16> { typedef uint16_t type; static __device__ __forceinline__ uint16_t cvt(float f) { return f2bf(f); } };

__device__ __forceinline__ void store_y(void* y, int y_dtype, int64_t o, float v) {
    if (y_dtype == SQ_BF16) reinterpret_cast<uint16_t*>(y)[o] = f2bf(v);
    else if (y_dtype == SQ_F16) reinterpret_cast<uint16_t*>(y)[o] = f2h(v);
    else reinterpret_cast<float*>(y)[o] = v;
}

// Tag j of a row's little-endian bit stream (any width 1..16).  `W` bounds the second word.
__device__ __forceinline__ uint32_t tag_at(const uint32_t* __restrict__ row, int W, int bits, int j) {
    const int p = j * bits, w = p >> 5, s = p & 31;
    const uint32_t lo = row[w];
    const uint32_t hi = (s + bits > 32 && w + 1 < W) ? row[w + 1] : 0u;
    const uint64_t v = ((uint64_t)hi << 32) | lo;
    return (uint32_t)(v >> s) & ((1u << bits) - 1u);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// A caller's workspace starts with SQ_WS_HEADER bytes that only the tag-stream kernel touches: the partial sums its
// workgroups exchange.  Every word of them is zero whenever no call is running (a partial sum doubles as its own arrival
// flag and whoever adds it up puts zero back), so they must be zero when the workspace is first handed over and nothing
// else may ever be written there; the other launchers get the part behind the header.
constexpr size_t SQ_WS_HEADER = (size_t)32 << 20;
// The partial sums fill at most the first SQ_WS_SUMS bytes of the header; its last page holds the error word of the
// exchange (at SQ_WS_ERR_OFF): set by a workgroup that gave up waiting for a partial sum, read by every later launch
// (which then writes NaN everywhere: partial sums that arrive late leave the header dirty, and a dirty header must
// never yield finite numbers), cleared by sq_workspace_reset.
constexpr size_t SQ_WS_SUMS = SQ_WS_HEADER - 4096;
constexpr size_t SQ_WS_ERR_OFF = SQ_WS_HEADER - 256;

// error plumbing shared by the launchers (defined in sq_api.hip)
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);
int device_cus();       // compute units of the current device (cached)

// launchers implemented in the kernel translation units
int launch_dequant(const sq_matrix& m, void* out, int out_dtype, int64_t ld_out, int r0, int r1, hipStream_t s,
                   bool raw = false);
int launch_small(const sq_matrix* mats, int n, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                 int64_t ldy, int B, void* ws, size_t ws_bytes, void* sums, hipStream_t s,
                 const sq_producer* from = nullptr);
// one activation row of these pieces is a single launch of the tag-stream kernel, which can produce its own x
bool small_fuses_producer(const sq_matrix* mats, int n, int B);
// the two pieces are a gate and an up projection whose launch can write SiLU(gate) * up itself
bool small_fuses_silu(const sq_matrix* mats, int n, int B);
int launch_small_silu(const sq_matrix* mats, int n, const void* x, int x_dtype, int64_t ldx, void* act, int64_t ld_act, int B,
                      void* sums, hipStream_t s, const sq_producer* from = nullptr);
size_t small_workspace(const sq_matrix* mats, int n, int B);
// some piece runs the tag-stream kernel, whose partial sums live in the workspace header (`sums` above)
bool small_uses_sums(const sq_matrix* mats, int n);
int launch_gemm(const sq_matrix* mats, int n, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                int64_t ldy, int T, void* ws, size_t ws_bytes, void* sums, hipStream_t s);
// stacks with column orders and more than a few activation rows: sq_linear_small runs the decode + tile GEMM route
bool small_takes_gemm_route(const sq_matrix* mats, int n, int B, const void* x, int64_t ldx);
size_t small_gemm_route_workspace(const sq_matrix* mats, int n, int B);
// most activation rows for which passes of SQ_SMALL_BMAX rows through the decode-time kernel beat decode + GEMM
// for these pieces (0: never)
int small_pass_limit(const sq_matrix* mats, int n);
size_t gemm_workspace(const sq_matrix* mats, int n, int T);
int launch_gemm_dense(const void* w, int w_dtype, int64_t ldw, int R, int C, const void* x, int x_dtype, int64_t ldx,
                      void* y, int y_dtype, int64_t ldy, int T, hipStream_t s, void* ws = nullptr, size_t ws_bytes = 0);
size_t gemm_dense_workspace(int R, int C, int T);

// d = 4 / 12-bit pieces at 1 or 2 activation rows, from the file's row-major tags (sq_segs.hip)
bool segs_shape(const sq_matrix& m);
bool segs_fits(const sq_matrix* mats, int cnt, int B, int cus);
int launch_segs_group(const sq_matrix* mats, int cnt, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                      int64_t ldy, int B, int cus, hipStream_t s);

// tile-major copy of the tags for the matrix-core decode kernel (host routines, sq_gemv.hip)
bool tiled_format_ok(int R, int W, int C, int d, int bits);
size_t tiled_bytes(int R, int W);
void tiled_build(const uint32_t* tags, int R, int W, int bits, uint32_t* out);

// the block-32 side formats (8-bit output head, 4-bit embedding)
int launch_q8_small(const int8_t* q, const uint16_t* sc, int V, int C, const void* x, int x_dtype, int64_t ldx, void* y,
                    int y_dtype, int64_t ldy, int B, hipStream_t s);
bool q8_mid(int C, int B);                  // 3 .. 320 activation rows (C % 256 == 0) on MFMA passes of up to 64
size_t q8_mid_workspace(int C, int B);
int launch_q8_mid(const int8_t* q, const uint16_t* sc, int V, int C, const void* x, int x_dtype, int64_t ldx, void* y,
                  int y_dtype, int64_t ldy, int B, void* ws, size_t ws_bytes, hipStream_t s);
size_t q8_workspace(int V, int C, int T);
int launch_q8_large(const int8_t* q, const uint16_t* sc, int V, int C, const void* x, int x_dtype, int64_t ldx, void* y,
                    int y_dtype, int64_t ldy, int T, void* ws, size_t ws_bytes, hipStream_t s);
int launch_q8_dequant(const int8_t* q, const uint16_t* sc, int C, void* out, int out_dtype, int64_t ld_out, int r0, int r1,
                      hipStream_t s);
int launch_q4_embed(const uint8_t* q, const uint16_t* sc, int V, int C, const int64_t* ids, int64_t n_ids, void* out,
                    int out_dtype, int64_t ld_out, hipStream_t s);

// elementwise neighbours of the decode-time products (sq_neighbours.hip)
int launch_addnorm(const float* h_in, float* h_out, int64_t ld_h, const void* add, int add_dtype, int64_t ld_add, const void* w,
                   int w_dtype, const int32_t* perms, int M, int B, int C, float eps, void* out, int out_dtype, hipStream_t s);
int launch_silu_mul(const void* gate, const void* up, int dtype, int64_t ld, const int32_t* perms, int M, int B, int C, void* out,
                    hipStream_t s);

}  // namespace sq
