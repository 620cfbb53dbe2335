// extern "C" surface of libsqhip.so: argument checks, error text, dispatch to the launchers.
#include <algorithm>
#include <atomic>
#include <stdarg.h>
#include <stdio.h>
#include "sq_stream.h"

namespace sq {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SQ_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
    return SQ_OK;
}

int device_cus() {
    static int cus[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cus[dev] == 0) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
        cus[dev] = v;
    }
    return cus[dev];
}

static int check_matrix(const sq_matrix& m, const char* who) {
    if (!m.table || !m.row_scale) return fail(SQ_EINVAL, "%s: null table/row_scale", who);
    if (!m.tags && !stream_shape(m)) return fail(SQ_EINVAL, "%s: null tags (only a matrix with a slice stream may drop them)", who);
    if (m.R < 0 || m.C <= 0 || m.d <= 0 || m.C % m.d) return fail(SQ_EINVAL, "%s: R %d C %d d %d", who, m.R, m.C, m.d);
    if (m.bits < 1 || m.bits > 16) return fail(SQ_EINVAL, "%s: tag bits %d outside 1..16", who, m.bits);
    if (m.G < 1 || m.G > 256 || (m.G > 1 && !m.row_book)) return fail(SQ_EINVAL, "%s: G %d needs row_book", who, m.G);
    if (m.M > 1 && (!m.row_mask || !m.perms)) return fail(SQ_EINVAL, "%s: M %d needs row_mask and perms", who, m.M);
    if (m.M > 256) return fail(SQ_EINVAL, "%s: M %d > 256", who, m.M);
    if ((int64_t)m.W * 32 < (int64_t)(m.C / m.d) * m.bits) return fail(SQ_EINVAL, "%s: W %d too small", who, m.W);
    if (((uintptr_t)m.tags & 3) || ((uintptr_t)m.table & 1) || ((uintptr_t)m.row_scale & 1))
        return fail(SQ_EINVAL, "%s: misaligned tensor", who);
    if ((m.d * 2) % 8 == 0 && ((uintptr_t)m.table & 15)) return fail(SQ_EINVAL, "%s: table must be 16-byte aligned", who);
    return SQ_OK;
}

static int check_xy(const char* who, const sq_matrix* mats, int n, const void* x, int x_dtype, int64_t ldx, const void* y,
                    int y_dtype, int64_t ldy, int rows) {
    if (n < 0 || (n > 0 && !mats)) return fail(SQ_EINVAL, "%s: n_mats %d", who, n);
    if (rows < 0) return fail(SQ_EINVAL, "%s: %d activation rows", who, rows);
    if (x_dtype != SQ_F16 && x_dtype != SQ_BF16) return fail(SQ_EINVAL, "%s: x_dtype %d", who, x_dtype);
    if (y_dtype != SQ_F16 && y_dtype != SQ_BF16 && y_dtype != SQ_F32) return fail(SQ_EINVAL, "%s: y_dtype %d", who, y_dtype);
    if (y_dtype != SQ_F32 && y_dtype != x_dtype) return fail(SQ_EINVAL, "%s: y_dtype %d != x_dtype %d", who, y_dtype, x_dtype);
    if (rows > 0 && n > 0 && (!x || !y)) return fail(SQ_EINVAL, "%s: null x / y", who);
    int64_t need = 0;
    for (int i = 0; i < n; ++i) {
        int rc = check_matrix(mats[i], who);
        if (rc) return rc;
        if (mats[i].C != mats[0].C) return fail(SQ_EINVAL, "%s: stacked pieces disagree on the input size (%d vs %d)", who, mats[i].C, mats[0].C);
        if (mats[i].y_off < 0) return fail(SQ_EINVAL, "%s: y_off %d", who, mats[i].y_off);
        if ((int64_t)mats[i].y_off + mats[i].R > need) need = (int64_t)mats[i].y_off + mats[i].R;
    }
    if (n > 0 && rows > 1 && (ldx < mats[0].C || ldy < need)) return fail(SQ_EINVAL, "%s: ldx %lld / ldy %lld too small", who, (long long)ldx, (long long)ldy);
    return SQ_OK;
}

}  // namespace sq

using namespace sq;

extern "C" {

int sq_version(void) { return 109; }

const char* sq_last_error(void) { return g_err; }

int sq_dequant(const sq_matrix* m, void* out, int out_dtype, int64_t ld_out, int32_t r0, int32_t r1, void* stream) {
    if (!m) return fail(SQ_EINVAL, "sq_dequant: null matrix");
    int rc = check_matrix(*m, "sq_dequant");
    if (rc) return rc;
    if (r0 < 0 || r1 < r0 || r1 > m->R) return fail(SQ_EINVAL, "sq_dequant: rows [%d, %d) outside [0, %d)", r0, r1, m->R);
    if (r1 == r0) return SQ_OK;
    if (!out || ld_out < m->C) return fail(SQ_EINVAL, "sq_dequant: out %p ld_out %lld", out, (long long)ld_out);
    return launch_dequant(*m, out, out_dtype, ld_out, r0, r1, (hipStream_t)stream);
}

// A workspace as the launchers see it: the header (partial sums of the tag-stream kernel) and what lies behind it.  A
// buffer of at least SQ_WS_HEADER bytes always begins with the header; a smaller one has none and is used from its
// first byte, which serves pieces that keep no partial sums (a private workspace of a few KB for a d = 4 matrix).
struct WsParts { void* sums; char* inner; size_t inner_bytes; };
static WsParts split_workspace(void* workspace, size_t ws_bytes) {
    if (!workspace) return WsParts{nullptr, nullptr, 0};
    if (ws_bytes >= SQ_WS_HEADER) return WsParts{workspace, (char*)workspace + SQ_WS_HEADER, ws_bytes - SQ_WS_HEADER};
    return WsParts{nullptr, (char*)workspace, ws_bytes};
}

// The exchange of the tag-stream kernel gave up in an earlier launch on this device (its workgroups set a host-visible
// word then): partial sums may have arrived late, the header is no longer known to be zero, and every launch on it
// writes NaN until sq_workspace_reset has run.
static int refuse_if_poisoned(const char* who, const sq_matrix* mats, int n) {
    if (small_uses_sums(mats, n) && stream_host_flag_set())
        return fail(SQ_ELAUNCH, "%s: an earlier launch on this device gave up waiting for a partial sum; its workspace header may be "
                                "dirty: call sq_workspace_reset on the workspace before using it again", who);
    return SQ_OK;
}

int sq_linear_small(const sq_matrix* mats, int32_t n_mats, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                    int64_t ldy, int32_t B, void* workspace, size_t ws_bytes, void* stream) {
    int rc = check_xy("sq_linear_small", mats, n_mats, x, x_dtype, ldx, y, y_dtype, ldy, B);
    if (rc) return rc;
    if (B > SQ_SMALL_BMAX) return fail(SQ_EINVAL, "sq_linear_small: B %d > %d", B, SQ_SMALL_BMAX);
    if (B == 0 || n_mats == 0) return SQ_OK;
    if ((rc = refuse_if_poisoned("sq_linear_small", mats, n_mats))) return rc;
    const WsParts w = split_workspace(workspace, ws_bytes);
    if (w.sums) (void)stream_host_flag((hipStream_t)stream, true);      // (one pinned host word per device, first call only)
    if (small_takes_gemm_route(mats, n_mats, B, x, ldx))
        return launch_gemm(mats, n_mats, x, x_dtype, ldx, y, y_dtype, ldy, B, w.inner, w.inner_bytes, w.sums, (hipStream_t)stream);
    return launch_small(mats, n_mats, x, x_dtype, ldx, y, y_dtype, ldy, B, w.inner, w.inner_bytes, w.sums, (hipStream_t)stream);
}

// ---- sq_linear_small for callers that cannot allocate: the workspace is a device array of this library.
// In host code `g_static_scratch` is only a handle for hipGetSymbolAddress: the device address it stands for is looked
// up once per device and kept; kernels are handed that address, never the symbol.
static_assert(sq::SQ_WS_HEADER == SQ_WS_HEADER_BYTES, "the header size is part of the ABI");
static __device__ __align__(256) unsigned char g_static_scratch[SQ_NOALLOC_SCRATCH_BYTES];
static std::atomic<void*> g_static_scratch_ptr[64];

// This device's copy of the scratch array (its address, looked up on first use with the device current), or nullptr +
// error.  The array is zero when the code object is loaded, which is what the header must be before the first call:
// nothing is launched here, so a first call under stream capture records only the product's own kernels.  (Two
// threads that race to the first call look the same address up twice.)
static void* static_scratch() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { fail(SQ_ELAUNCH, "sq_linear_small_noalloc: no current device"); return nullptr; }
    void* ptr = g_static_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_scratch));
        if (e != hipSuccess || !ptr) { fail(SQ_ELAUNCH, "sq_linear_small_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e)); return nullptr; }
        g_static_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    return ptr;
}

int sq_linear_small_noalloc(const sq_matrix* mats, int32_t n_mats, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                            int64_t ldy, int32_t B, void* stream) {
    int rc = check_xy("sq_linear_small_noalloc", mats, n_mats, x, x_dtype, ldx, y, y_dtype, ldy, B);
    if (rc) return rc;
    if (B > SQ_SMALL_BMAX) return fail(SQ_EINVAL, "sq_linear_small_noalloc: B %d > %d", B, SQ_SMALL_BMAX);
    if (B == 0 || n_mats == 0) return SQ_OK;
    const size_t need = sq_workspace_bytes(mats, n_mats, B, 0);
    if (need > (size_t)SQ_NOALLOC_SCRATCH_BYTES)
        return fail(SQ_EWORKSPACE, "sq_linear_small_noalloc: these pieces need %zu bytes of workspace at %d rows, the built-in scratch holds %u "
                                   "(use sq_linear_small with a workspace of the caller's)", need, B, (unsigned)SQ_NOALLOC_SCRATCH_BYTES);
    if ((rc = refuse_if_poisoned("sq_linear_small_noalloc", mats, n_mats))) return rc;
    char* ws = (char*)static_scratch();
    if (!ws) return SQ_ELAUNCH;
    const size_t inner = (size_t)SQ_NOALLOC_SCRATCH_BYTES - SQ_WS_HEADER;
    if (small_takes_gemm_route(mats, n_mats, B, x, ldx))
        return launch_gemm(mats, n_mats, x, x_dtype, ldx, y, y_dtype, ldy, B, ws + SQ_WS_HEADER, inner, ws, (hipStream_t)stream);
    return launch_small(mats, n_mats, x, x_dtype, ldx, y, y_dtype, ldy, B, ws + SQ_WS_HEADER, inner, ws, (hipStream_t)stream);
}

int sq_linear_small_from(const sq_matrix* mats, int32_t n_mats, const sq_producer* from, int x_dtype, void* y, int y_dtype,
                         int64_t ldy, int32_t B, void* workspace, size_t ws_bytes, void* stream) {
    const char* who = "sq_linear_small_from";
    if (!from) return fail(SQ_EINVAL, "%s: null producer", who);
    if (from->mode != SQ_FROM_ADDNORM && from->mode != SQ_FROM_SILU_MUL) return fail(SQ_EINVAL, "%s: mode %d", who, from->mode);
    int rc = check_xy(who, mats, n_mats, from->x_out, x_dtype, n_mats > 0 ? mats[0].C : 0, y, y_dtype, ldy, B);
    if (rc) return rc;
    if (B > SQ_SMALL_BMAX) return fail(SQ_EINVAL, "%s: B %d > %d", who, B, SQ_SMALL_BMAX);
    if (B == 0 || n_mats == 0) return SQ_OK;
    const int C = mats[0].C;
    const bool addnorm = from->mode == SQ_FROM_ADDNORM;
    if (C % 8 || ((uintptr_t)from->x_out & 15)) return fail(SQ_EINVAL, "%s: x_out must be 16-byte aligned and C %% 8 == 0", who);
    if (addnorm && (!from->h_in || !from->w)) return fail(SQ_EINVAL, "%s: null h_in / w", who);
    if (addnorm && from->h_out == from->h_in) return fail(SQ_EINVAL, "%s: h_out must not be h_in", who);
    {
        // workgroups read the producer's operands while others already write x_out / h_out: no overlap allowed
        auto overlap = [](const void* p, size_t n, const void* q, size_t m) {
            return p && q && (const char*)p < (const char*)q + m && (const char*)q < (const char*)p + n;
        };
        const size_t xo = (size_t)B * C * 2, in16 = ((size_t)(B - 1) * (size_t)(B > 1 ? from->ld_in : 0) + C) * 2;
        const size_t h32 = ((size_t)(B - 1) * (size_t)(B > 1 ? from->ld_h : 0) + C) * 4;
        if (overlap(from->x_out, xo, from->add, in16) || overlap(from->x_out, xo, from->up, in16) ||
            (addnorm && (overlap(from->x_out, xo, from->h_in, h32) || overlap(from->x_out, xo, from->w, (size_t)C * 2) ||
                         overlap(from->h_out, h32, from->add, in16) || overlap(from->h_out, h32, from->h_in, h32))))
            return fail(SQ_EINVAL, "%s: x_out / h_out must not overlap the producer's operands", who);
    }
    if (!addnorm && (!from->add || !from->up)) return fail(SQ_EINVAL, "%s: null gate / up", who);
    if (B > 1 && ((addnorm && from->ld_h < C) || ((from->add || !addnorm) && from->ld_in < C)))
        return fail(SQ_EINVAL, "%s: ld_h %lld / ld_in %lld too small", who, (long long)from->ld_h, (long long)from->ld_in);
    hipStream_t s = (hipStream_t)stream;
    if ((rc = refuse_if_poisoned(who, mats, n_mats))) return rc;
    const WsParts wp = split_workspace(workspace, ws_bytes);
    const bool has_ws = wp.sums != nullptr;
    void* ws = wp.inner;
    const size_t wsb = wp.inner_bytes;
    if (has_ws) (void)stream_host_flag(s, true);
    const bool aligned = (((uintptr_t)from->h_in | (uintptr_t)from->h_out | (uintptr_t)from->add | (uintptr_t)from->up | (uintptr_t)from->w) & 15) == 0;
    if (addnorm && aligned && small_fuses_producer(mats, n_mats, B))
        return launch_small(mats, n_mats, from->x_out, x_dtype, C, y, y_dtype, ldy, B, ws, wsb, has_ws ? workspace : nullptr, s, from);
    rc = addnorm ? launch_addnorm(from->h_in, from->h_out, from->ld_h, from->add, x_dtype, from->ld_in, from->w, x_dtype, nullptr, 1, B,
                                  C, from->eps, from->x_out, x_dtype, s)
                 : launch_silu_mul(from->add, from->up, x_dtype, from->ld_in, nullptr, 1, B, C, from->x_out, s);
    if (rc) return rc;
    if (small_takes_gemm_route(mats, n_mats, B, from->x_out, C))
        return launch_gemm(mats, n_mats, from->x_out, x_dtype, C, y, y_dtype, ldy, B, ws, wsb, has_ws ? workspace : nullptr, s);
    return launch_small(mats, n_mats, from->x_out, x_dtype, C, y, y_dtype, ldy, B, ws, wsb, has_ws ? workspace : nullptr, s);
}

int sq_linear_small_silu(const sq_matrix* mats, int32_t n_mats, const sq_producer* from, const void* x, int dtype, int64_t ldx,
                         void* out, int64_t ld_out, int32_t B, void* workspace, size_t ws_bytes, void* stream) {
    const char* who = "sq_linear_small_silu";
    if (n_mats != 2 || !mats) return fail(SQ_EINVAL, "%s: the gate and the up piece, n_mats %d", who, n_mats);
    if (from && from->mode != SQ_FROM_ADDNORM) return fail(SQ_EINVAL, "%s: producer mode %d", who, from->mode);
    const void* xin = from ? from->x_out : x;
    const int64_t ldxin = from ? mats[0].C : ldx;
    // (check_xy's bound on ldy is for the stacked y, which is not written here: ld_out is checked below)
    int rc = check_xy(who, mats, n_mats, xin, dtype, ldxin, out, dtype, (int64_t)1 << 40, B);
    if (rc) return rc;
    if (mats[0].R != mats[1].R) return fail(SQ_EINVAL, "%s: gate has %d rows, up %d", who, mats[0].R, mats[1].R);
    if (B > 1 && ld_out < mats[0].R) return fail(SQ_EINVAL, "%s: ld_out %lld < %d", who, (long long)ld_out, mats[0].R);
    if (B == 0) return SQ_OK;
    if (from && (B != 1 || !from->h_in || !from->w || from->h_out == from->h_in || (mats[0].C % 8) || ((uintptr_t)from->x_out & 15)))
        return fail(SQ_EINVAL, "%s: a fused producer takes one activation row, h_in and w, h_out != h_in, a 16-byte aligned x_out", who);
    if ((rc = refuse_if_poisoned(who, mats, n_mats))) return rc;
    const WsParts wp = split_workspace(workspace, ws_bytes);
    hipStream_t s = (hipStream_t)stream;
    if (wp.sums) (void)stream_host_flag(s, true);
    return launch_small_silu(mats, n_mats, xin, dtype, ldxin, out, ld_out, B, wp.sums ? workspace : nullptr, s, from);
}

int sq_linear_gemm(const sq_matrix* mats, int32_t n_mats, const void* x, int x_dtype, int64_t ldx, void* y, int y_dtype,
                   int64_t ldy, int32_t T, void* workspace, size_t ws_bytes, void* stream) {
    int rc = check_xy("sq_linear_gemm", mats, n_mats, x, x_dtype, ldx, y, y_dtype, ldy, T);
    if (rc) return rc;
    if (T == 0 || n_mats == 0) return SQ_OK;
    if (T <= SQ_SMALL_BMAX && (rc = refuse_if_poisoned("sq_linear_gemm", mats, n_mats))) return rc;
    const WsParts w = split_workspace(workspace, ws_bytes);
    return launch_gemm(mats, n_mats, x, x_dtype, ldx, y, y_dtype, ldy, T, w.inner, w.inner_bytes, w.sums, (hipStream_t)stream);
}

int sq_gemm_dense(const void* w, int w_dtype, int64_t ldw, int32_t R, int32_t C, const void* x, int x_dtype, int64_t ldx,
                  void* y, int y_dtype, int64_t ldy, int32_t T, void* stream) {
    if (x_dtype != SQ_F16 && x_dtype != SQ_BF16) return fail(SQ_EINVAL, "sq_gemm_dense: x_dtype %d", x_dtype);
    if (w_dtype != SQ_F16 && w_dtype != SQ_BF16) return fail(SQ_EINVAL, "sq_gemm_dense: w_dtype %d", w_dtype);
    if (y_dtype != SQ_F32 && y_dtype != SQ_F16 && y_dtype != SQ_BF16) return fail(SQ_EINVAL, "sq_gemm_dense: y_dtype %d", y_dtype);
    if (R < 0 || C <= 0 || T < 0) return fail(SQ_EINVAL, "sq_gemm_dense: R %d C %d T %d", R, C, T);
    if (R == 0 || T == 0) return SQ_OK;
    if (!w || !x || !y || ldw < C || ldx < C || ldy < R) return fail(SQ_EINVAL, "sq_gemm_dense: bad pointer or stride");
    return launch_gemm_dense(w, w_dtype, ldw, R, C, x, x_dtype, ldx, y, y_dtype, ldy, T, (hipStream_t)stream);
}

int sq_gemm_dense_ws(const void* w, int w_dtype, int64_t ldw, int32_t R, int32_t C, const void* x, int x_dtype, int64_t ldx,
                     void* y, int y_dtype, int64_t ldy, int32_t T, void* workspace, size_t ws_bytes, void* stream) {
    if (!workspace || ws_bytes <= SQ_WS_HEADER || ((uintptr_t)workspace & 255))
        return sq_gemm_dense(w, w_dtype, ldw, R, C, x, x_dtype, ldx, y, y_dtype, ldy, T, stream);
    if (x_dtype != SQ_F16 && x_dtype != SQ_BF16) return fail(SQ_EINVAL, "sq_gemm_dense_ws: x_dtype %d", x_dtype);
    if (w_dtype != SQ_F16 && w_dtype != SQ_BF16) return fail(SQ_EINVAL, "sq_gemm_dense_ws: w_dtype %d", w_dtype);
    if (y_dtype != SQ_F32 && y_dtype != SQ_F16 && y_dtype != SQ_BF16) return fail(SQ_EINVAL, "sq_gemm_dense_ws: y_dtype %d", y_dtype);
    if (R < 0 || C <= 0 || T < 0) return fail(SQ_EINVAL, "sq_gemm_dense_ws: R %d C %d T %d", R, C, T);
    if (R == 0 || T == 0) return SQ_OK;
    if (!w || !x || !y || ldw < C || ldx < C || ldy < R) return fail(SQ_EINVAL, "sq_gemm_dense_ws: bad pointer or stride");
    return launch_gemm_dense(w, w_dtype, ldw, R, C, x, x_dtype, ldx, y, y_dtype, ldy, T, (hipStream_t)stream,
                             (char*)workspace + SQ_WS_HEADER, ws_bytes - SQ_WS_HEADER);
}

size_t sq_gemm_dense_workspace_bytes(int32_t R, int32_t C, int32_t T) {
    if (R <= 0 || C <= 0 || T <= 0) return 0;
    const size_t inner = gemm_dense_workspace(R, C, T);
    return inner ? inner + SQ_WS_HEADER : 0;
}

size_t sq_workspace_bytes(const sq_matrix* mats, int32_t n_mats, int32_t rows, int which) {
    if (!mats || n_mats <= 0 || rows <= 0) return 0;
    // which & 1 = 0 covers both kernels a stack with column orders may take (the caller's x decides, see sq_linear_small)
    const size_t inner = (which & 1) == 0 ? std::max(small_workspace(mats, n_mats, rows), small_gemm_route_workspace(mats, n_mats, rows))
                                          : gemm_workspace(mats, n_mats, rows);
    const bool sums = small_uses_sums(mats, n_mats);
    // which & 2: a workspace of the caller's own for these pieces alone: no header unless they keep partial sums in
    // it (or need so much that the buffer would be taken for one that begins with a header)
    if ((which & 2) && !sums && inner < SQ_WS_HEADER) return inner;
    return (inner || sums) ? inner + SQ_WS_HEADER : 0;
}

__global__ void workspace_clear_kernel(uint32_t* p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

int sq_workspace_reset(void* workspace, size_t ws_bytes, void* stream) {
    if (!workspace || ((uintptr_t)workspace & 255)) return fail(SQ_EINVAL, "sq_workspace_reset: workspace %p", workspace);
    if (ws_bytes < SQ_WS_HEADER) return SQ_OK;                  // no header, nothing to clear
    const size_t n = SQ_WS_HEADER / 4;
    hipLaunchKernelGGL(workspace_clear_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, (uint32_t*)workspace, n);
    int rc = check_launch("sq_workspace_reset");
    if (rc) return rc;
    stream_host_flag_clear();
    return SQ_OK;
}

int sq_workspace_status(const void* workspace, size_t ws_bytes, void* stream) {
    if (!workspace) return fail(SQ_EINVAL, "sq_workspace_status: null workspace");
    if (ws_bytes < SQ_WS_HEADER) return SQ_OK;
    uint32_t word = 0;
    hipError_t e = hipMemcpyAsync(&word, (const char*)workspace + SQ_WS_ERR_OFF, 4, hipMemcpyDeviceToHost, (hipStream_t)stream);
    if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return fail(SQ_ELAUNCH, "sq_workspace_status: %s", hipGetErrorString(e));
    if (word) return fail(SQ_ELAUNCH, "sq_workspace_status: a launch on this workspace gave up waiting for a partial sum; results since "
                                      "then are NaN: call sq_workspace_reset");
    return SQ_OK;
}

void sq_stream_spin_limit(int32_t polls) { stream_set_spin(polls); }

int sq_noalloc_reset(void* stream) {
    char* ws = (char*)static_scratch();
    if (!ws) return SQ_ELAUNCH;
    return sq_workspace_reset(ws, (size_t)SQ_NOALLOC_SCRATCH_BYTES, stream);
}

size_t sq_stream_bytes_balanced(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits,
                                const uint8_t* row_mask_host, int32_t runs, const void* table_host) {
    if (!tags_host || d <= 0 || (int64_t)W * 32 < (int64_t)(C / d) * bits) return 0;
    if (!stream_format_ok(R, C, d, bits)) return !row_mask_host && tiled_format_ok(R, W, C, d, bits) ? tiled_bytes(R, W) : 0;
    return stream_bytes_host((const uint32_t*)tags_host, R, W, C, d, bits, row_mask_host, runs, (const uint16_t*)table_host);
}

int sq_stream_build_balanced(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits,
                             const uint8_t* row_mask_host, int32_t runs, const void* table_host, void* out_host, size_t out_bytes,
                             int32_t* runs_out, int32_t* groups_out) {
    if (!tags_host || !out_host || !runs_out || !groups_out) return fail(SQ_EINVAL, "sq_stream_build: null pointer");
    if (d > 0 && !stream_format_ok(R, C, d, bits) && !row_mask_host && tiled_format_ok(R, W, C, d, bits)) {
        if (out_bytes < tiled_bytes(R, W)) return fail(SQ_EINVAL, "sq_stream_build: out_bytes %zu < %zu", out_bytes, tiled_bytes(R, W));
        tiled_build((const uint32_t*)tags_host, R, W, bits, (uint32_t*)out_host);
        *runs_out = 0;
        *groups_out = 0;
        return SQ_OK;
    }
    if (d <= 0 || !stream_format_ok(R, C, d, bits)) return fail(SQ_EUNSUPPORTED, "sq_stream_build: d %d bits %d R %d not covered", d, bits, R);
    if ((int64_t)W * 32 < (int64_t)(C / d) * bits) return fail(SQ_EINVAL, "sq_stream_build: W %d too small", W);
    return stream_build_host((const uint32_t*)tags_host, R, W, C, d, bits, row_mask_host, runs, (unsigned char*)out_host,
                             out_bytes, runs_out, groups_out, (const uint16_t*)table_host);
}

int sq_codebook_balance(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits, uint16_t* remap_out) {
    if (!tags_host || !remap_out) return fail(SQ_EINVAL, "sq_codebook_balance: null pointer");
    if (d <= 0 || !stream_format_ok(R, C, d, bits)) return fail(SQ_EUNSUPPORTED, "sq_codebook_balance: d %d bits %d R %d not covered", d, bits, R);
    if ((int64_t)W * 32 < (int64_t)(C / d) * bits) return fail(SQ_EINVAL, "sq_codebook_balance: W %d too small", W);
    stream_balance_host((const uint32_t*)tags_host, R, W, C, d, bits, remap_out);
    return SQ_OK;
}

// ---- several codebooks per matrix: the labels of the tag stream are book << bits | tag (sq_stream.h)
static int books_check(const char* who, int32_t R, int32_t G, const uint8_t* row_book_host) {
    if (G < 1 || G > 256 || (G & (G - 1)) != 0) return fail(SQ_EUNSUPPORTED, "%s: %d codebooks (a power of two is needed)", who, G);
    if (G > 1 && !row_book_host) return fail(SQ_EINVAL, "%s: G %d needs row_book", who, G);
    if (G > 1)
        for (int32_t r = 0; r < R; ++r)
            if (row_book_host[r] >= G) return fail(SQ_EINVAL, "%s: row %d names codebook %d of %d", who, r, (int)row_book_host[r], G);
    return SQ_OK;
}

size_t sq_stream_bytes_books(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits, int32_t G,
                             const uint8_t* row_book_host, const uint8_t* row_mask_host, int32_t runs) {
    // (one codebook, and the formats whose buffer is the tile-major copy of the tags, which does not depend on the codebooks)
    if (G <= 1 || (d > 0 && !stream_format_ok(R, C, d, bits, G) && !row_mask_host && tiled_format_ok(R, W, C, d, bits)))
        return sq_stream_bytes_balanced(tags_host, R, W, C, d, bits, row_mask_host, runs, nullptr);
    if (!tags_host || d <= 0 || R <= 0 || (int64_t)W * 32 < (int64_t)(C / d) * bits) return 0;
    if (!stream_format_ok(R, C, d, bits, G) || books_check("sq_stream_bytes_books", R, G, row_book_host) != SQ_OK) return 0;
    return stream_bytes_host((const uint32_t*)tags_host, R, W, C, d, bits, row_mask_host, runs, nullptr, G, row_book_host);
}

int sq_stream_build_books(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits, int32_t G,
                          const uint8_t* row_book_host, const uint8_t* row_mask_host, int32_t runs, void* out_host,
                          size_t out_bytes, int32_t* runs_out, int32_t* groups_out) {
    if (G <= 1 || (d > 0 && !stream_format_ok(R, C, d, bits, G) && !row_mask_host && tiled_format_ok(R, W, C, d, bits)))
        return sq_stream_build_balanced(tags_host, R, W, C, d, bits, row_mask_host, runs, nullptr, out_host, out_bytes, runs_out, groups_out);
    if (!tags_host || !out_host || !runs_out || !groups_out) return fail(SQ_EINVAL, "sq_stream_build_books: null pointer");
    if (d <= 0 || !stream_format_ok(R, C, d, bits, G))
        return fail(SQ_EUNSUPPORTED, "sq_stream_build_books: d %d bits %d G %d R %d not covered", d, bits, G, R);
    if ((int64_t)W * 32 < (int64_t)(C / d) * bits) return fail(SQ_EINVAL, "sq_stream_build_books: W %d too small", W);
    if (int rc = books_check("sq_stream_build_books", R, G, row_book_host)) return rc;
    return stream_build_host((const uint32_t*)tags_host, R, W, C, d, bits, row_mask_host, runs, (unsigned char*)out_host,
                             out_bytes, runs_out, groups_out, nullptr, G, row_book_host);
}

int sq_codebook_balance_books(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits, int32_t G,
                              const uint8_t* row_book_host, uint16_t* remap_out) {
    if (!tags_host || !remap_out) return fail(SQ_EINVAL, "sq_codebook_balance_books: null pointer");
    if (d <= 0 || !stream_format_ok(R, C, d, bits, G))
        return fail(SQ_EUNSUPPORTED, "sq_codebook_balance_books: d %d bits %d G %d R %d not covered", d, bits, G, R);
    if ((int64_t)W * 32 < (int64_t)(C / d) * bits) return fail(SQ_EINVAL, "sq_codebook_balance_books: W %d too small", W);
    if (int rc = books_check("sq_codebook_balance_books", R, G, row_book_host)) return rc;
    stream_balance_host((const uint32_t*)tags_host, R, W, C, d, bits, remap_out, G, G > 1 ? row_book_host : nullptr);
    return SQ_OK;
}

size_t sq_stream_bytes(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits,
                       const uint8_t* row_mask_host, int32_t runs) {
    return sq_stream_bytes_balanced(tags_host, R, W, C, d, bits, row_mask_host, runs, nullptr);
}

int sq_stream_build(const int32_t* tags_host, int32_t R, int32_t W, int32_t C, int32_t d, int32_t bits,
                    const uint8_t* row_mask_host, int32_t runs, void* out_host, size_t out_bytes, int32_t* runs_out,
                    int32_t* groups_out) {
    return sq_stream_build_balanced(tags_host, R, W, C, d, bits, row_mask_host, runs, nullptr, out_host, out_bytes, runs_out, groups_out);
}

static int check_q8(const char* who, const void* q, const void* scale, int32_t V, int32_t C) {
    if (V < 0 || C <= 0 || C % 32) return fail(SQ_EINVAL, "%s: V %d C %d (C must be a positive multiple of 32)", who, V, C);
    if (V > 0 && (!q || !scale)) return fail(SQ_EINVAL, "%s: null q / scale", who);
    if (((uintptr_t)q & 15) || ((uintptr_t)scale & 15)) return fail(SQ_EINVAL, "%s: q and scale must be 16-byte aligned", who);
    return SQ_OK;
}

int sq_q8_linear(const int8_t* q, const uint16_t* scale, int32_t V, int32_t C, const void* x, int x_dtype, int64_t ldx,
                 void* y, int y_dtype, int64_t ldy, int32_t B, void* workspace, size_t ws_bytes, void* stream) {
    int rc = check_q8("sq_q8_linear", q, scale, V, C);
    if (rc) return rc;
    if (B < 0) return fail(SQ_EINVAL, "sq_q8_linear: %d activation rows", B);
    if (x_dtype != SQ_F16 && x_dtype != SQ_BF16) return fail(SQ_EINVAL, "sq_q8_linear: x_dtype %d", x_dtype);
    if (y_dtype != SQ_F16 && y_dtype != SQ_BF16 && y_dtype != SQ_F32) return fail(SQ_EINVAL, "sq_q8_linear: y_dtype %d", y_dtype);
    if (y_dtype != SQ_F32 && y_dtype != x_dtype) return fail(SQ_EINVAL, "sq_q8_linear: y_dtype %d != x_dtype %d", y_dtype, x_dtype);
    if (B == 0 || V == 0) return SQ_OK;
    if (!x || !y) return fail(SQ_EINVAL, "sq_q8_linear: null x / y");
    if (B > 1 && (ldx < C || ldy < V)) return fail(SQ_EINVAL, "sq_q8_linear: ldx %lld / ldy %lld too small", (long long)ldx, (long long)ldy);
    const bool has_ws = workspace && ws_bytes >= SQ_WS_HEADER;
    if (q8_mid(C, B))
        return launch_q8_mid(q, scale, V, C, x, x_dtype, ldx, y, y_dtype, ldy, B, has_ws ? (char*)workspace + SQ_WS_HEADER : nullptr,
                             has_ws ? ws_bytes - SQ_WS_HEADER : 0, (hipStream_t)stream);
    if (B <= SQ_SMALL_BMAX) return launch_q8_small(q, scale, V, C, x, x_dtype, ldx, y, y_dtype, ldy, B, (hipStream_t)stream);
    return launch_q8_large(q, scale, V, C, x, x_dtype, ldx, y, y_dtype, ldy, B, has_ws ? (char*)workspace + SQ_WS_HEADER : nullptr,
                           has_ws ? ws_bytes - SQ_WS_HEADER : 0, (hipStream_t)stream);
}

size_t sq_q8_workspace_bytes(int32_t V, int32_t C, int32_t B) {
    if (C <= 0 || C % 32) return 0;
    const size_t inner = q8_mid(C, B) ? q8_mid_workspace(C, B) : q8_workspace(V, C, B);
    return inner ? inner + SQ_WS_HEADER : 0;
}

int sq_q8_dequant(const int8_t* q, const uint16_t* scale, int32_t V, int32_t C, void* out, int out_dtype, int64_t ld_out,
                  int32_t r0, int32_t r1, void* stream) {
    int rc = check_q8("sq_q8_dequant", q, scale, V, C);
    if (rc) return rc;
    if (out_dtype != SQ_F16 && out_dtype != SQ_BF16 && out_dtype != SQ_F32) return fail(SQ_EINVAL, "sq_q8_dequant: out_dtype %d", out_dtype);
    if (r0 < 0 || r1 < r0 || r1 > V) return fail(SQ_EINVAL, "sq_q8_dequant: rows [%d, %d) outside [0, %d)", r0, r1, V);
    if (r1 == r0) return SQ_OK;
    if (!out || ld_out < C) return fail(SQ_EINVAL, "sq_q8_dequant: out %p ld_out %lld", out, (long long)ld_out);
    return launch_q8_dequant(q, scale, C, out, out_dtype, ld_out, r0, r1, (hipStream_t)stream);
}

int sq_q4_embed(const uint8_t* q, const uint16_t* scale, int32_t V, int32_t C, const int64_t* ids, int64_t n_ids, void* out,
                int out_dtype, int64_t ld_out, void* stream) {
    int rc = check_q8("sq_q4_embed", q, scale, V, C);
    if (rc) return rc;
    if (out_dtype != SQ_F16 && out_dtype != SQ_BF16 && out_dtype != SQ_F32) return fail(SQ_EINVAL, "sq_q4_embed: out_dtype %d", out_dtype);
    if (n_ids < 0) return fail(SQ_EINVAL, "sq_q4_embed: %lld ids", (long long)n_ids);
    if (n_ids == 0) return SQ_OK;
    if (!ids || !out || ld_out < C) return fail(SQ_EINVAL, "sq_q4_embed: ids %p out %p ld_out %lld", (const void*)ids, out, (long long)ld_out);
    if ((uintptr_t)ids & 7) return fail(SQ_EINVAL, "sq_q4_embed: ids must be 8-byte aligned");
    return launch_q4_embed(q, scale, V, C, ids, n_ids, out, out_dtype, ld_out, (hipStream_t)stream);
}

static bool is16(int dt) { return dt == SQ_F16 || dt == SQ_BF16; }

int sq_addnorm(const float* h_in, float* h_out, int64_t ld_h, const void* add, int add_dtype, int64_t ld_add, const void* w,
               int w_dtype, const int32_t* perms, int32_t M, int32_t B, int32_t C, float eps, void* out, int out_dtype,
               void* stream) {
    if (B < 0 || C <= 0) return fail(SQ_EINVAL, "sq_addnorm: B %d C %d", B, C);
    if (!is16(w_dtype) || !is16(out_dtype) || (add && !is16(add_dtype)))
        return fail(SQ_EINVAL, "sq_addnorm: add / w / out must be fp16 or bf16 (%d / %d / %d)", add_dtype, w_dtype, out_dtype);
    if (perms && M <= 0) return fail(SQ_EINVAL, "sq_addnorm: %d column orders", M);
    if (B == 0) return SQ_OK;
    if (!h_in || !w || !out) return fail(SQ_EINVAL, "sq_addnorm: null h_in / w / out");
    if (B > 1 && (ld_h < C || (add && ld_add < C))) return fail(SQ_EINVAL, "sq_addnorm: ld_h %lld / ld_add %lld too small", (long long)ld_h, (long long)ld_add);
    if (perms && h_out == h_in) return fail(SQ_EINVAL, "sq_addnorm: with column orders h_out must not be h_in");
    return launch_addnorm(h_in, h_out, ld_h, add, add_dtype, ld_add, w, w_dtype, perms, M, B, C, eps, out, out_dtype, (hipStream_t)stream);
}

int sq_silu_mul(const void* gate, const void* up, int dtype, int64_t ld, const int32_t* perms, int32_t M, int32_t B, int32_t C,
                void* out, void* stream) {
    if (B < 0 || C <= 0) return fail(SQ_EINVAL, "sq_silu_mul: B %d C %d", B, C);
    if (!is16(dtype)) return fail(SQ_EINVAL, "sq_silu_mul: dtype %d", dtype);
    if (perms && M <= 0) return fail(SQ_EINVAL, "sq_silu_mul: %d column orders", M);
    if (B == 0) return SQ_OK;
    if (!gate || !up || !out) return fail(SQ_EINVAL, "sq_silu_mul: null gate / up / out");
    if (B > 1 && ld < C) return fail(SQ_EINVAL, "sq_silu_mul: ld %lld too small", (long long)ld);
    return launch_silu_mul(gate, up, dtype, ld, perms, M, B, C, out, (hipStream_t)stream);
}

}  // extern "C"
