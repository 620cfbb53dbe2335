// Dense decode of a packed codebook matrix: one thread per chunk.
//   out[r, perm[mask[r]][j*d + k]] = rn_T( f32(table[book[r]*K + tag[r, j]][k]) * f32(row_scale[r]) )
// The fp32 product of two fp16 values is exact, so T = fp32 reproduces the CPU decode bit
// for bit and T = fp16 / bf16 differ from it by exactly one round-to-nearest-even.
#include "sq_stream.h"

namespace sq {

template <int DT, int D>   // D = 0: any chunk width (scalar path)
__global__ __launch_bounds__(256) void dequant_kernel(sq_matrix m, typename store_as<DT>::type* __restrict__ out,
                                                      int64_t ld_out, int r0, int r1, int raw) {
    typedef typename store_as<DT>::type T;
    const int d = D ? D : m.d;
    const int nch = m.C / d;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)(r1 - r0) * nch) return;
    const int rr = (int)(idx / nch), j = (int)(idx - (int64_t)rr * nch);
    const int r = r0 + rr;
    const uint32_t* row = reinterpret_cast<const uint32_t*>(m.tags) + (int64_t)r * m.W;
    uint32_t tag = tag_at(row, m.W, m.bits, j);
    if (m.row_book) tag += (uint32_t)m.row_book[r] << m.bits;
    const float s = raw ? 1.f : h2f(m.row_scale[r]);     // raw: unscaled codewords (exact in fp16)
    const uint16_t* cw = m.table + (int64_t)tag * d;
    T* o = out + (int64_t)rr * ld_out;
    // a perms array without row_mask is one matrix-wide column order
    const int32_t* pm = m.perms ? m.perms + (int64_t)(m.row_mask ? m.row_mask[r] : 0) * m.C : nullptr;
    if (D == 8 && !pm) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(cw);
        T t[8];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            t[2 * k] = store_as<DT>::cvt(h2f((uint16_t)(v[k] & 0xFFFFu)) * s);
            t[2 * k + 1] = store_as<DT>::cvt(h2f((uint16_t)(v[k] >> 16)) * s);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) o[j * 8 + k] = t[k];
        return;
    }
    if (D == 4 && !pm) {
        const u32x2 v = *reinterpret_cast<const u32x2*>(cw);
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            o[j * 4 + 2 * k] = store_as<DT>::cvt(h2f((uint16_t)(v[k] & 0xFFFFu)) * s);
            o[j * 4 + 2 * k + 1] = store_as<DT>::cvt(h2f((uint16_t)(v[k] >> 16)) * s);
        }
        return;
    }
    for (int k = 0; k < d; ++k) {
        const int c = j * d + k;
        o[pm ? pm[c] : c] = store_as<DT>::cvt(h2f(cw[k]) * s);
    }
}

// d = 8 without column orders: four chunks per thread, 256 chunks apart, so that a thread has four tag loads and then
// four 16-byte table gathers in flight instead of one (the decode is bound by the rate and latency of those gathers,
// which hit L2, not HBM).  Same arithmetic as dequant_kernel; `vec`: 16-byte aligned rows of a 16-bit type, stored
// as one 16-byte piece per chunk; raw fp16 output copies the codeword's bits.
template <int DT>
__device__ __forceinline__ void dequant8x4_block(const sq_matrix& m, typename store_as<DT>::type* __restrict__ out, int64_t ld_out,
                                                 int r0, int r1, int raw, int vec, int block) {
    typedef typename store_as<DT>::type T;
    const int nch = m.C / 8;
    const int total = (r1 - r0) * nch;                          // < 2^31, checked by the launcher
    const int base = block * 1024 + (int)threadIdx.x;
    int rr[4], j[4];
    bool ok[4];
    uint32_t tag[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        int idx = base + k * 256;
        ok[k] = idx < total;
        idx = min(idx, total - 1);
        rr[k] = idx / nch;
        j[k] = idx - rr[k] * nch;
        const uint32_t* row = reinterpret_cast<const uint32_t*>(m.tags) + (int64_t)(r0 + rr[k]) * m.W;
        tag[k] = tag_at(row, m.W, m.bits, j[k]);
    }
    if (m.row_book) {
#pragma unroll
        for (int k = 0; k < 4; ++k) tag[k] += (uint32_t)m.row_book[r0 + rr[k]] << m.bits;
    }
    u32x4 cw[4];
    float s[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        cw[k] = *reinterpret_cast<const u32x4*>(m.table + (int64_t)tag[k] * 8);
        s[k] = raw ? 1.f : h2f(m.row_scale[r0 + rr[k]]);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        if (!ok[k]) continue;
        T* o = out + (int64_t)rr[k] * ld_out + j[k] * 8;
        if (DT == SQ_F16 && raw && vec) {
            *reinterpret_cast<u32x4*>(o) = cw[k];
            continue;
        }
        T t[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            t[2 * e] = store_as<DT>::cvt(h2f((uint16_t)(cw[k][e] & 0xFFFFu)) * s[k]);
            t[2 * e + 1] = store_as<DT>::cvt(h2f((uint16_t)(cw[k][e] >> 16)) * s[k]);
        }
        if (DT != SQ_F32 && vec) {
            u32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = (uint32_t)t[2 * e] | ((uint32_t)t[2 * e + 1] << 16);
            *reinterpret_cast<u32x4*>(o) = v;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = t[e];
        }
    }
}

template <int DT>
__global__ __launch_bounds__(256) void dequant8x4_kernel(sq_matrix m, typename store_as<DT>::type* __restrict__ out,
                                                         int64_t ld_out, int r0, int r1, int raw, int vec) {
    dequant8x4_block<DT>(m, out, ld_out, r0, r1, raw, vec, (int)blockIdx.x);
}

// The raw fp16 decode of a whole matrix and the fp16 copy of a bf16 activation matrix in one launch: the decode is
// bound by table gathers out of L2, the copy by HBM, so the copy's `nc` workgroups (8 elements per thread) are dealt
// evenly among the decode's `nd` and the two overlap instead of running one after the other.
__global__ __launch_bounds__(256) void dequant8x4_cvt_kernel(sq_matrix m, uint16_t* __restrict__ out, int64_t ld_out,
                                                             const uint16_t* __restrict__ x, int64_t ldx, int T, int C,
                                                             uint16_t* __restrict__ xout, int nd, int nc) {
    const int64_t b = blockIdx.x, total = (int64_t)nd + nc;
    const int cb = (int)(b * nc / total);                       // copy workgroups before this one
    if ((int)((b + 1) * nc / total) == cb) {
        dequant8x4_block<SQ_F16>(m, out, ld_out, 0, m.R, 1, 1, (int)b - cb);
        return;
    }
    const int64_t i = ((int64_t)cb * 256 + threadIdx.x) * 8;
    if (i >= (int64_t)T * C) return;
    const int t = (int)(i / C), c = (int)(i - (int64_t)t * C);
    u32x4 v = *reinterpret_cast<const u32x4*>(x + (int64_t)t * ldx + c);
    v.x = bf2h_x2(v.x); v.y = bf2h_x2(v.y); v.z = bf2h_x2(v.z); v.w = bf2h_x2(v.w);
    *reinterpret_cast<u32x4*>(xout + i) = v;
}

// Matrices with column orders: scattering 2-byte values straight to HBM costs 4x the plain decode, so a
// workgroup decodes one row at a time into LDS at its permuted positions (ds_write of one element each, the
// order read as whole 16/32-byte pieces) and then writes the row out in 16-byte pieces.
template <int DT, int D>   // D = 8 or 4
__global__ __launch_bounds__(256) void dequant_rows_lds_kernel(sq_matrix m, typename store_as<DT>::type* __restrict__ out,
                                                               int64_t ld_out, int r0, int r1, int raw, int vec_out) {
    typedef typename store_as<DT>::type T;
    extern __shared__ __attribute__((aligned(16))) unsigned char row_smem[];
    T* row_lds = reinterpret_cast<T*>(row_smem);
    const int C = m.C, nch = C / D, tid = threadIdx.x;
    constexpr int V = 16 / (int)sizeof(T);              // elements per 16-byte store
    for (int r = r0 + blockIdx.x; r < r1; r += gridDim.x) {
        const uint32_t* row = reinterpret_cast<const uint32_t*>(m.tags) + (int64_t)r * m.W;
        const uint32_t boff = m.row_book ? (uint32_t)m.row_book[r] << m.bits : 0u;
        const float s = raw ? 1.f : h2f(m.row_scale[r]);
        const int32_t* pm = m.perms + (int64_t)(m.row_mask ? m.row_mask[r] : 0) * C;
        for (int j = tid; j < nch; j += 256) {
            const uint32_t tag = tag_at(row, m.W, m.bits, j) + boff;
            const uint16_t* cw = m.table + (int64_t)tag * D;
            uint32_t v[D / 2];
            int32_t p[D];
            if (D == 8) {
                const u32x4 t = *reinterpret_cast<const u32x4*>(cw);
                v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3];
                const u32x4 p0 = *reinterpret_cast<const u32x4*>(pm + j * 8), p1 = *reinterpret_cast<const u32x4*>(pm + j * 8 + 4);
#pragma unroll
                for (int k = 0; k < 4; ++k) { p[k] = (int32_t)p0[k]; p[4 + k] = (int32_t)p1[k]; }
            } else {
                const u32x2 t = *reinterpret_cast<const u32x2*>(cw);
                v[0] = t[0]; v[1] = t[1];
                const u32x4 p0 = *reinterpret_cast<const u32x4*>(pm + j * 4);
#pragma unroll
                for (int k = 0; k < 4; ++k) p[k] = (int32_t)p0[k];
            }
#pragma unroll
            for (int k = 0; k < D / 2; ++k) {
                row_lds[p[2 * k]] = store_as<DT>::cvt(h2f((uint16_t)(v[k] & 0xFFFFu)) * s);
                row_lds[p[2 * k + 1]] = store_as<DT>::cvt(h2f((uint16_t)(v[k] >> 16)) * s);
            }
        }
        __syncthreads();
        T* o = out + (int64_t)(r - r0) * ld_out;
        if (vec_out) {
            for (int c = tid * V; c < C; c += 256 * V)
                *reinterpret_cast<u32x4*>(o + c) = *reinterpret_cast<const u32x4*>(row_lds + c);
        } else {
            for (int c = tid; c < C; c += 256) o[c] = row_lds[c];
        }
        __syncthreads();
    }
}

static bool dequant8x4_ok(const sq_matrix& m, int64_t n) {
    return m.d == 8 && !m.perms && n > 0 && n < ((int64_t)1 << 31) - 1024 && ((uintptr_t)m.table & 15) == 0;
}

template <int DT>
static int launch_dt(const sq_matrix& m, void* out, int64_t ld_out, int r0, int r1, hipStream_t s, int raw) {
    typedef typename store_as<DT>::type T;
    const int64_t n = (int64_t)(r1 - r0) * (m.C / m.d);
    if (n == 0) return SQ_OK;
    const size_t row_bytes = (size_t)m.C * sizeof(T);
    if (m.perms && (m.d == 8 || m.d == 4) && row_bytes <= 65536 && ((uintptr_t)m.perms & 15) == 0 && ((uintptr_t)m.table & 15) == 0 &&
        m.C % 4 == 0) {
        constexpr int V = 16 / (int)sizeof(T);
        const int vec_out = ((uintptr_t)out & 15) == 0 && ld_out % V == 0 && m.C % V == 0;
        const int per_cu = (int)(131072 / row_bytes) < 8 ? (int)(131072 / row_bytes) : 8;       // workgroups that share a CU's LDS
        const int want = device_cus() * (per_cu < 1 ? 1 : per_cu);
        const unsigned rgrid = (unsigned)(r1 - r0 < want ? r1 - r0 : want);
        if (m.d == 8) hipLaunchKernelGGL((dequant_rows_lds_kernel<DT, 8>), dim3(rgrid), dim3(256), row_bytes, s, m, (T*)out, ld_out, r0, r1, raw, vec_out);
        else hipLaunchKernelGGL((dequant_rows_lds_kernel<DT, 4>), dim3(rgrid), dim3(256), row_bytes, s, m, (T*)out, ld_out, r0, r1, raw, vec_out);
        return check_launch("sq_dequant");
    }
    if (dequant8x4_ok(m, n)) {
        const int vec = sizeof(T) == 2 && ((uintptr_t)out & 15) == 0 && ld_out % 8 == 0;
        hipLaunchKernelGGL((dequant8x4_kernel<DT>), dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, s, m, (T*)out, ld_out, r0, r1, raw, vec);
        return check_launch("sq_dequant");
    }
    const unsigned grid = (unsigned)((n + 255) / 256);
    if (m.d == 8) hipLaunchKernelGGL((dequant_kernel<DT, 8>), dim3(grid), dim3(256), 0, s, m, (T*)out, ld_out, r0, r1, raw);
    else if (m.d == 4) hipLaunchKernelGGL((dequant_kernel<DT, 4>), dim3(grid), dim3(256), 0, s, m, (T*)out, ld_out, r0, r1, raw);
    else hipLaunchKernelGGL((dequant_kernel<DT, 0>), dim3(grid), dim3(256), 0, s, m, (T*)out, ld_out, r0, r1, raw);
    return check_launch("sq_dequant");
}

// Raw fp16 decode of every row of `m` into out[r * ld_out + c] together with the fp16 copy of the bf16 matrix x
// [T, C] (row stride ldx, 16-byte aligned rows, C % 8 == 0) into xout [T, C].  Returns 1 without launching
// anything when the matrix does not take the four-chunk kernel; the caller then launches the two steps itself.
int launch_dequant_with_cvt(const sq_matrix& m, void* out, int64_t ld_out, const uint16_t* x, int64_t ldx, int T, int C,
                            uint16_t* xout, hipStream_t s) {
    const int64_t n = (int64_t)m.R * (m.C / (m.d ? m.d : 1)), ne = (int64_t)T * C;
    if (!m.tags || !dequant8x4_ok(m, n) || ((uintptr_t)out & 15) || ld_out % 8 || ne <= 0 || ne >= ((int64_t)1 << 40)) return 1;
    const int64_t nd = (n + 1023) / 1024, nc = (ne / 8 + 255) / 256;
    if (nd + nc >= ((int64_t)1 << 31)) return 1;
    hipLaunchKernelGGL(dequant8x4_cvt_kernel, dim3((unsigned)(nd + nc)), dim3(256), 0, s, m, (uint16_t*)out, ld_out, x, ldx, T, C, xout,
                       (int)nd, (int)nc);
    return check_launch("sq_linear_gemm(decode + fp16 copy)");
}

int launch_dequant(const sq_matrix& m, void* out, int out_dtype, int64_t ld_out, int r0, int r1, hipStream_t s, bool raw) {
    if (!m.tags) return launch_stream_dequant(m, out, out_dtype, ld_out, r0, r1, s, raw);    // one-copy residency
    switch (out_dtype) {
        case SQ_F32: return launch_dt<SQ_F32>(m, out, ld_out, r0, r1, s, raw ? 1 : 0);
        case SQ_F16: return launch_dt<SQ_F16>(m, out, ld_out, r0, r1, s, raw ? 1 : 0);
        case SQ_BF16: return launch_dt<SQ_BF16>(m, out, ld_out, r0, r1, s, raw ? 1 : 0);
    }
    return fail(SQ_EINVAL, "sq_dequant: out_dtype %d", out_dtype);
}

}  // namespace sq
