// The packed file's two block-32 side formats on the device:
//   8-bit output head   q int8  [V, C],   scale fp16 [V, C/32]:  w[v, c] = q[v, c] * scale[v, c/32]
//   4-bit embedding     q uint8 [V, C/2], scale fp16 [V, C/32]:  w[v, 2k]   = ((q[v, k] & 15) - 8) * scale[v, 2k/32]
//                                                                w[v, 2k+1] = ((q[v, k] >> 4) - 8) * scale[v, (2k+1)/32]
// (reference shapequant/packed.py:30-40, 134-159).  The head product Y[b, v] = sum_c X[b, c] * w[v, c] is pure
// weight streaming for a handful of activation rows: every byte of q is read once from HBM and nothing is
// reused, so the kernel is built around full-line loads (one wave load = 1 KB of one weight row), many loads in
// flight per wave, and as few VALU operations per weight byte as the fp16 dot-product instruction allows.
#include "sq_common.h"

namespace sq {

constexpr int Q8_WAVE_ROWS = 8;                 // weight rows a wave carries at once (loads in flight, x reuse)
constexpr int Q8_WG_WAVES = 4;
constexpr int Q8_TASK_ROWS = Q8_WAVE_ROWS * Q8_WG_WAVES;
constexpr int Q8_LDS_HALVES = 32768;            // fp16 activations a workgroup stages (64 KB)

struct Q8Args {
    const int8_t* q;
    const uint16_t* sc;
    const uint16_t* x;
    void* y;
    int64_t ldx, ldy;
    int V, C, B, x_dtype, y_dtype, tasks, x_vec;
};

// Four int8 -> two half2, exactly: flip the sign bit (q + 128 as a byte), put the byte under the exponent of
// 1024 (0x6400 | u = 1024 + u) and subtract 1152.
__device__ __forceinline__ void i8x4_to_h2(uint32_t w, half2v& lo, half2v& hi) {
    const uint32_t u = w ^ 0x80808080u;
    const half2v bias = {(half_t)1152.f, (half_t)1152.f};
    // v_perm_b32: selector bytes 0..3 pick from the second operand, 4..7 from the first
    lo = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - bias;
    hi = __builtin_bit_cast(half2v, __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - bias;
}

// Sums N per-lane values over the 64 lanes with N - 1 + log2(64 / N) exchanges instead of 6 N: each halving step
// trades half of the values with the lane `o` away.  Afterwards lane l holds the total of value l >> (6 - log2 N)
// (in v[0]).
template <int N>
__device__ __forceinline__ void wave_sum_many(float (&v)[N], int lane) {
    int o = 32;
#pragma unroll
    for (int n = N; n > 1; n >>= 1, o >>= 1) {
        // bitwise select on a lane mask: a ?: on the array elements is turned into a select of the INDEX,
        // i.e. dynamic indexing of a register array
        const uint32_t up = (lane & o) ? 0xFFFFFFFFu : 0u;
#pragma unroll
        for (int i = 0; i < n / 2; ++i) {
            const uint32_t a = __builtin_bit_cast(uint32_t, v[i]), b = __builtin_bit_cast(uint32_t, v[i + n / 2]);
            const float give = __builtin_bit_cast(float, (a & up) | (b & ~up));
            const float keep = __builtin_bit_cast(float, (b & up) | (a & ~up));
            v[i] = keep + __shfl_xor(give, o, 64);
        }
    }
#pragma unroll
    for (; o > 0; o >>= 1) v[0] += __shfl_xor(v[0], o, 64);
}

template <int N> struct log2_of { static constexpr int value = 1 + log2_of<N / 2>::value; };
template <> struct log2_of<1> { static constexpr int value = 0; };

struct Q8Regs {
    u32x4 w[Q8_WAVE_ROWS];
    uint16_t s[Q8_WAVE_ROWS];
};

// One wave load per row: 16 bytes per lane at column step*1024 + lane*16 (clamped inside the row), and the
// scale of that lane's block.  Uniform row base + 32-bit lane offset keeps the addresses in few registers.
__device__ __forceinline__ void q8_load(Q8Regs& r, const Q8Args& a, int row0, int col) {
    const int nblk = a.C >> 5;
#pragma unroll
    for (int i = 0; i < Q8_WAVE_ROWS; ++i) {
        const int row = min(row0 + i, a.V - 1);
        const int8_t* base = a.q + (int64_t)row * a.C;
        r.w[i] = *reinterpret_cast<const u32x4*>(base + col);
        r.s[i] = a.sc[(int64_t)row * nblk + (col >> 5)];
    }
}

// Persistent workgroups of 4 waves; a task is 32 consecutive rows (8 per wave).  The NB activation rows sit in LDS
// as fp16 for the whole launch.  Each wave walks its rows' columns 1 KB at a time with the next step's loads
// (possibly the next task's first step) issued before the current step is multiplied.
template <int NB>
__global__ __launch_bounds__(256, 2) void q8_gemv_kernel(Q8Args a) {
    extern __shared__ __attribute__((aligned(16))) uint16_t xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int C = a.C;
    if (a.x_vec) {
        for (int i = tid * 8; i < NB * C; i += 256 * 8) {
            const int nb = i / C, c = i - nb * C;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (nb < a.B) {
                v = *reinterpret_cast<const u32x4*>(a.x + nb * a.ldx + c);
                if (a.x_dtype == SQ_BF16) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) v[k] = bf2h_x2(v[k]);
                }
            }
            *reinterpret_cast<u32x4*>(xs + i) = v;
        }
    } else {
        for (int i = tid; i < NB * C; i += 256) {
            const int nb = i / C, c = i - nb * C;
            uint16_t v = 0;
            if (nb < a.B) {
                v = a.x[nb * a.ldx + c];
                if (a.x_dtype == SQ_BF16) v = __builtin_bit_cast(uint16_t, bf2h(v));
            }
            xs[i] = v;
        }
    }
    __syncthreads();

    const int nsteps = (C + 1023) >> 10;
    int task = blockIdx.x, step = 0;
    if (task >= a.tasks) return;
    float acc[Q8_WAVE_ROWS * NB];
#pragma unroll
    for (int i = 0; i < Q8_WAVE_ROWS * NB; ++i) acc[i] = 0.f;
    Q8Regs cur, nxt;
    {
        const int col = lane * 16;
        q8_load(cur, a, task * Q8_TASK_ROWS + wave * Q8_WAVE_ROWS, col < C ? col : C - 16);
    }
    nxt = cur;
    while (task < a.tasks) {
        int ntask = task, nstep = step + 1;
        if (nstep == nsteps) { nstep = 0; ntask += gridDim.x; }
        if (ntask < a.tasks) {
            const int col = nstep * 1024 + lane * 16;
            q8_load(nxt, a, ntask * Q8_TASK_ROWS + wave * Q8_WAVE_ROWS, col < C ? col : C - 16);
        }
        {
            const int col = step * 1024 + lane * 16;
            const bool live = col < C;
            const int cc = live ? col : C - 16;
            half2v xf[NB][8];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const u32x4 lo = *reinterpret_cast<const u32x4*>(xs + nb * C + cc);
                const u32x4 hi = *reinterpret_cast<const u32x4*>(xs + nb * C + cc + 8);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t l = lo[k], h = hi[k];
                    xf[nb][k] = __builtin_bit_cast(half2v, l);
                    xf[nb][4 + k] = __builtin_bit_cast(half2v, h);
                }
            }
#pragma unroll
            for (int i = 0; i < Q8_WAVE_ROWS; ++i) {
                half2v wh[8];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t wk = cur.w[i][k];
                    i8x4_to_h2(wk, wh[2 * k], wh[2 * k + 1]);
                }
                const float sc = live ? h2f(cur.s[i]) : 0.f;
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    float d = 0.f;
#pragma unroll
                    for (int k = 0; k < 8; ++k) d = __builtin_amdgcn_fdot2(wh[k], xf[nb][k], d, false);
                    acc[i * NB + nb] += d * sc;
                }
            }
        }
        if (nstep == 0) {
            wave_sum_many<Q8_WAVE_ROWS * NB>(acc, lane);
            constexpr int SH = 6 - log2_of<Q8_WAVE_ROWS * NB>::value;
            const int idx = lane >> SH;
            const int i = idx / NB, nb = idx - i * NB;
            const int row = task * Q8_TASK_ROWS + wave * Q8_WAVE_ROWS + i;
            if ((lane & ((1 << SH) - 1)) == 0 && row < a.V && nb < a.B) store_y(a.y, a.y_dtype, nb * a.ldy + row, acc[0]);
#pragma unroll
            for (int k = 0; k < Q8_WAVE_ROWS * NB; ++k) acc[k] = 0.f;
        }
        cur = nxt;
        task = ntask;
        step = nstep;
    }
}

// Rows [r0, r1) as dense values, one 16-byte load (16 weights, half a block) per thread.
template <int DT>
__global__ __launch_bounds__(256) void q8_dequant_kernel(const int8_t* __restrict__ q, const uint16_t* __restrict__ sc,
                                                         int C, typename store_as<DT>::type* __restrict__ out,
                                                         int64_t ld_out, int r0, int64_t n16) {
    typedef typename store_as<DT>::type T;
    const int per_row = C >> 4;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < n16; t += (int64_t)gridDim.x * 256) {
        const int rr = (int)(t / per_row), c = (int)(t - (int64_t)rr * per_row) * 16;
        const int64_t row = r0 + rr;
        const u32x4 v = *reinterpret_cast<const u32x4*>(q + row * C + c);
        const float s = h2f(sc[row * (C >> 5) + (c >> 5)]);
        T o[16];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t w = v[k];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[4 * k + e] = store_as<DT>::cvt((float)(int8_t)(w >> (8 * e)) * s);
        }
        T* dst = out + (int64_t)rr * ld_out + c;
#pragma unroll
        for (int k = 0; k < 16; ++k) dst[k] = o[k];
    }
}

// Embedding rows: one 16-byte load (32 weights, one block) per thread.  Ids outside [0, V) give a row of zeros.
template <int DT>
__global__ __launch_bounds__(256) void q4_embed_kernel(const uint8_t* __restrict__ q, const uint16_t* __restrict__ sc,
                                                       int V, int C, const int64_t* __restrict__ ids, int64_t n_ids,
                                                       typename store_as<DT>::type* __restrict__ out, int64_t ld_out) {
    typedef typename store_as<DT>::type T;
    const int nblk = C >> 5;
    const int64_t total = n_ids * nblk;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < total; t += (int64_t)gridDim.x * 256) {
        const int64_t i = t / nblk;
        const int b = (int)(t - i * nblk);
        const int64_t id = ids[i];
        T* dst = out + i * ld_out + b * 32;
        if (id < 0 || id >= V) {
#pragma unroll
            for (int k = 0; k < 32; ++k) dst[k] = store_as<DT>::cvt(0.f);
            continue;
        }
        const u32x4 v = *reinterpret_cast<const u32x4*>(q + id * (C >> 1) + b * 16);
        const float s = h2f(sc[id * nblk + b]);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t w = v[k];
#pragma unroll
            for (int e = 0; e < 8; ++e)
                dst[8 * k + e] = store_as<DT>::cvt((float)((int)((w >> (4 * e)) & 15u) - 8) * s);
        }
    }
}

static int q8_pass_rows(int B, int C) {
    int nb = B > 2 ? 4 : B > 1 ? 2 : 1;
    while (nb > 1 && nb * C > Q8_LDS_HALVES) nb >>= 1;
    return nb;
}

int launch_q8_small(const int8_t* q, const uint16_t* sc, int V, int C, const void* x, int x_dtype, int64_t ldx, void* y,
                    int y_dtype, int64_t ldy, int B, hipStream_t s) {
    if (C > Q8_LDS_HALVES) return fail(SQ_EUNSUPPORTED, "sq_q8_linear: C %d > %d", C, Q8_LDS_HALVES);
    const size_t ys = y_dtype == SQ_F32 ? 4 : 2;
    const int tasks = (V + Q8_TASK_ROWS - 1) / Q8_TASK_ROWS;
    const int max_wgs = 2 * device_cus();
    const int per = (tasks + max_wgs - 1) / max_wgs;
    const unsigned grid = (unsigned)((tasks + per - 1) / per);
    for (int b0 = 0; b0 < B;) {
        const int nb = q8_pass_rows(B - b0, C);
        Q8Args a{};
        a.q = q; a.sc = sc;
        a.x = (const uint16_t*)x + (int64_t)b0 * ldx;
        a.y = (char*)y + (size_t)b0 * ldy * ys;
        a.ldx = ldx; a.ldy = ldy; a.V = V; a.C = C;
        a.B = B - b0 < nb ? B - b0 : nb;
        a.x_dtype = x_dtype; a.y_dtype = y_dtype; a.tasks = tasks;
        a.x_vec = ((uintptr_t)a.x & 15) == 0 && (a.B == 1 || ldx % 8 == 0) && C % 8 == 0;
        const size_t lds = (size_t)nb * C * 2;
        if (nb == 4) hipLaunchKernelGGL(q8_gemv_kernel<4>, dim3(grid), dim3(256), lds, s, a);
        else if (nb == 2) hipLaunchKernelGGL(q8_gemv_kernel<2>, dim3(grid), dim3(256), lds, s, a);
        else hipLaunchKernelGGL(q8_gemv_kernel<1>, dim3(grid), dim3(256), lds, s, a);
        int rc = check_launch("q8_gemv_kernel");
        if (rc) return rc;
        b0 += a.B;
    }
    return SQ_OK;
}

int launch_q8_dequant(const int8_t* q, const uint16_t* sc, int C, void* out, int out_dtype, int64_t ld_out, int r0, int r1,
                      hipStream_t s) {
    const int64_t n16 = (int64_t)(r1 - r0) * (C >> 4);
    if (n16 == 0) return SQ_OK;
    const int64_t want = (n16 + 255) / 256;
    const unsigned grid = (unsigned)(want < 65536 ? want : 65536);
    if (out_dtype == SQ_F32)
        hipLaunchKernelGGL(q8_dequant_kernel<SQ_F32>, dim3(grid), dim3(256), 0, s, q, sc, C, (float*)out, ld_out, r0, n16);
    else if (out_dtype == SQ_F16)
        hipLaunchKernelGGL(q8_dequant_kernel<SQ_F16>, dim3(grid), dim3(256), 0, s, q, sc, C, (uint16_t*)out, ld_out, r0, n16);
    else
        hipLaunchKernelGGL(q8_dequant_kernel<SQ_BF16>, dim3(grid), dim3(256), 0, s, q, sc, C, (uint16_t*)out, ld_out, r0, n16);
    return check_launch("q8_dequant_kernel");
}

int launch_q4_embed(const uint8_t* q, const uint16_t* sc, int V, int C, const int64_t* ids, int64_t n_ids, void* out,
                    int out_dtype, int64_t ld_out, hipStream_t s) {
    const int64_t total = n_ids * (C >> 5);
    if (total == 0) return SQ_OK;
    const int64_t want = (total + 255) / 256;
    const unsigned grid = (unsigned)(want < 65536 ? want : 65536);
    if (out_dtype == SQ_F32)
        hipLaunchKernelGGL(q4_embed_kernel<SQ_F32>, dim3(grid), dim3(256), 0, s, q, sc, V, C, ids, n_ids, (float*)out, ld_out);
    else if (out_dtype == SQ_F16)
        hipLaunchKernelGGL(q4_embed_kernel<SQ_F16>, dim3(grid), dim3(256), 0, s, q, sc, V, C, ids, n_ids, (uint16_t*)out, ld_out);
    else
        hipLaunchKernelGGL(q4_embed_kernel<SQ_BF16>, dim3(grid), dim3(256), 0, s, q, sc, V, C, ids, n_ids, (uint16_t*)out, ld_out);
    return check_launch("q4_embed_kernel");
}

}  // namespace sq
