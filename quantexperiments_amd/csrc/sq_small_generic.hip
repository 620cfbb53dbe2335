// Any-shape decode-time product (fallback of sq_linear_small): one wave per output row,
// lanes stride over the row's chunks, up to NB activation rows per pass.  Handles every
// chunk width, tag width 1..16, mixture books and column orders; the specialised kernels in
// sq_gemv.hip take over for the shapes they cover.
#include "sq_common.h"

namespace sq {

struct GenericArgs {
    sq_matrix m[4];
    int row_end[4];   // prefix sums of R over the pieces
    int n;
    const uint16_t* x;
    int64_t ldx;
    void* y;
    int64_t ldy;
    int B;
};

template <int XDT> __device__ __forceinline__ float load_x(const uint16_t* p) { return XDT == SQ_F16 ? h2f(*p) : bf2f(*p); }

template <int XDT, int YDT, int NB>
__global__ __launch_bounds__(256) void small_generic_kernel(GenericArgs a) {
    typedef typename store_as<YDT>::type TY;
    const int lane = threadIdx.x & 63;
    const int g = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (g >= a.row_end[a.n - 1]) return;
    int p = 0;
    while (g >= a.row_end[p]) ++p;
    const sq_matrix& m = a.m[p];
    const int r = g - (p ? a.row_end[p - 1] : 0);
    const int d = m.d, nch = m.C / d;
    const uint32_t* row = reinterpret_cast<const uint32_t*>(m.tags) + (int64_t)r * m.W;
    const uint32_t boff = m.row_book ? (uint32_t)m.row_book[r] << m.bits : 0u;
    const int32_t* pm = m.perms ? m.perms + (int64_t)(m.row_mask ? m.row_mask[r] : 0) * m.C : nullptr;
    const float s = h2f(m.row_scale[r]);
    for (int b0 = 0; b0 < a.B; b0 += NB) {
        float acc[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[b] = 0.f;
        for (int j = lane; j < nch; j += 64) {
            const uint16_t* cw = m.table + (int64_t)(tag_at(row, m.W, m.bits, j) + boff) * d;
            for (int k = 0; k < d; ++k) {
                const float w = h2f(cw[k]);
                const int c = j * d + k;
                const int src = pm ? pm[c] : c;
#pragma unroll
                for (int b = 0; b < NB; ++b)
                    if (b0 + b < a.B) acc[b] = fmaf(w, load_x<XDT>(a.x + (int64_t)(b0 + b) * a.ldx + src), acc[b]);
            }
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const float v = wave_sum(acc[b]) * s;
            if (lane == 0 && b0 + b < a.B)
                reinterpret_cast<TY*>(a.y)[(int64_t)(b0 + b) * a.ldy + m.y_off + r] = store_as<YDT>::cvt(v);
        }
    }
}

template <int XDT, int YDT>
static int launch_xy(const GenericArgs& a, hipStream_t s) {
    const int rows = a.row_end[a.n - 1];
    const unsigned grid = (unsigned)((rows + 3) / 4);
    if (a.B == 1) hipLaunchKernelGGL((small_generic_kernel<XDT, YDT, 1>), dim3(grid), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((small_generic_kernel<XDT, YDT, 4>), dim3(grid), dim3(256), 0, s, a);
    return check_launch("sq_linear_small(generic)");
}

int launch_small_generic(const sq_matrix* mats, int n, const void* x, int x_dtype, int64_t ldx, void* y,
                         int y_dtype, int64_t ldy, int B, hipStream_t s) {
    for (int i0 = 0; i0 < n; i0 += 4) {
        GenericArgs a;
        a.n = n - i0 < 4 ? n - i0 : 4;
        int acc = 0;
        for (int i = 0; i < 4; ++i) {
            a.m[i] = mats[i0 + (i < a.n ? i : 0)];
            if (i < a.n) acc += a.m[i].R;
            a.row_end[i] = acc;
        }
        a.x = (const uint16_t*)x; a.ldx = ldx; a.y = y; a.ldy = ldy; a.B = B;
        if (acc == 0) continue;
        int rc;
#define SQ_GO(XD, YD) rc = launch_xy<XD, YD>(a, s)
        if (x_dtype == SQ_F16 && y_dtype == SQ_F16) SQ_GO(SQ_F16, SQ_F16);
        else if (x_dtype == SQ_F16 && y_dtype == SQ_F32) SQ_GO(SQ_F16, SQ_F32);
        else if (x_dtype == SQ_BF16 && y_dtype == SQ_BF16) SQ_GO(SQ_BF16, SQ_BF16);
        else if (x_dtype == SQ_BF16 && y_dtype == SQ_F32) SQ_GO(SQ_BF16, SQ_F32);
        else return fail(SQ_EINVAL, "sq_linear_small: x_dtype %d / y_dtype %d", x_dtype, y_dtype);
#undef SQ_GO
        if (rc) return rc;
    }
    return SQ_OK;
}

}  // namespace sq
