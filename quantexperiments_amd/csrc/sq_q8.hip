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

// ---- 3 .. Q8_MFMA_MAX_ROWS activation rows (C % 256 == 0): fp16 MFMA, 16, 32 or 64 activation rows per pass.
// v_mfma_f32_16x16x32_f16 operand layout: A: lane l supplies weight row l % 16, k = 8 * (l / 16) .. + 7; B: token
// l % 16, the same k; D: lane l holds token l % 16, weight rows 4 * (l / 16) .. + 3.  Weights are the A operand and a
// wave owns 16 rows.  The rows reach the wave through LDS: global_load_lds (no registers in between) fetches them in
// lane order ALONG the row, one instruction = 8 rows x 128 bytes, whole cache lines with 8 consecutive lanes per
// line, into a private ring of D steps per wave (a step = 16 rows x 128 columns = 2 KB); the wave reads its
// fragments back in the operand layout (lane (r, g) takes pieces 2 g and 2 g + 1 of row r, 32 bytes per step), so
// the weights need no barrier, only counted waits.  Rows are XOR-swizzled in 16-byte pieces (piece p of row r at
// slot p ^ ((r >> 1) & 7), applied through the source addresses of the copy), so the 16 lanes of an LDS read clock
// hit 16 different bank groups.  Block scales travel the same way (a 4-byte copy per lane: 16 bytes per row and
// chunk of 256 columns).  Each 16-byte piece feeds two MFMAs per block of 16 tokens; the k index of MFMA m of piece
// j is column 128 s + 16 (2 g + j) + 8 m + e, and the activations (B operand) are read with the same mapping from
// LDS, where the workgroup keeps the current 256-column chunk of the fp16 activations (global_load_lds, double
// buffered, one barrier per chunk).  The block scale is folded into the fp16 weight (one rounding, as the
// reference's tile kernel does, shapequant/kernels/batched_runs.py:442-447): all 16 weights of a piece sit in one
// block.  A first form loaded the operand layout straight from memory (lane = row, 16 bytes per lane): every
// quarter wave then touches 16 different cache lines, and it stayed at 4.1-4.4 TB/s where this one reaches
// 5.2-5.5 TB/s (the one-row kernel: 5.7); 32 rows per wave on the 32x32x16 instruction was slower still.
constexpr int Q8_MFMA_MAX_ROWS = 320;           // up to here passes of 64 beat decode + tile GEMM (152,064 x 3,584: 151 us per pass,
                                                // 5 passes 755 us against ~880; 8 passes 1208 against 961 at 512 rows)

// x [B, C] (fp16 or bf16, any stride) -> fp16 [B, C] contiguous.
__global__ __launch_bounds__(256) void q8_x_kernel(const uint16_t* __restrict__ x, int64_t ldx, int B, int C, int x_dtype,
                                                   uint16_t* __restrict__ out) {
    const int64_t n = (int64_t)B * C;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const int b = (int)(i / C), c = (int)(i - (int64_t)b * C);
        const uint16_t v = x[b * ldx + c];
        out[i] = x_dtype == SQ_BF16 ? __builtin_bit_cast(uint16_t, bf2h(v)) : v;
    }
}

struct Q8MfmaArgs {
    const int8_t* q;
    const uint16_t* sc;
    const uint16_t* xh;     // fp16 [B, ldxh], rows 16-byte aligned
    void* y;
    int64_t ldy;
    int ldxh;
    int V, C, B, y_dtype, tasks;
    int vec_y;              // y rows allow 8-byte stores of 16-bit results (y 8-byte aligned, ldy % 4 == 0)
};

constexpr int q8_vmcnt(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }   // wait on vmcnt only

// weights ring + scales of d - 1 chunks (with a ring of 4 steps the scales of chunk c + 2 are requested while chunk c
// is still being multiplied)
constexpr int q8l_wave_bytes(int d) { return d * 2048 + (d - 1) * 256; }
constexpr int q8l_lds_bytes(int nblk, int waves, int d, int xs) { return 2 * nblk * 16 * xs * 256 + waves * q8l_wave_bytes(d); }

// NBLK 16-token blocks, WAVES waves per workgroup, ring of D steps per wave (one being multiplied, D - 1 in flight),
// x chunks of XS steps (128 XS columns; the first 16 NBLK XS / 4 waves copy 4 / XS tokens of every chunk each)
template <int NBLK, int WAVES, int D, int XS>
__global__ __launch_bounds__(WAVES * 64, WAVES == 8 ? 2 : 1) void q8_mfma_kernel(Q8MfmaArgs a) {
    static_assert((D == 3 || D == 4) && (XS == 2 || (XS == 1 && D == 3)), "wait counts below are written out for these");
    constexpr int Q8L_D = D, Q8L_WAVE_BYTES = q8l_wave_bytes(D);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* xs = smem;                                   // [2][16 NBLK tokens][256 XS bytes]
    constexpr int XPITCH = XS * 256, XBUF = NBLK * 16 * XPITCH;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    unsigned char* wl = smem + 2 * XBUF + wave * Q8L_WAVE_BYTES;  // this wave's ring
    unsigned char* sl_ = wl + Q8L_D * 2048;                        // this wave's scales: [D - 1][16 rows][16 bytes]
    const int task_raw = blockIdx.x * WAVES + wave;
    const bool active = task_raw < a.tasks;
    const int task = active ? task_raw : a.tasks - 1;
    const int r = lane & 15, g = lane >> 4;
    const int C = a.C, nblk = C >> 5, nsteps = C >> 7, nchunks = nsteps / XS;

    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    // activations: one copy instruction moves 1 KB = 4 / XS tokens of a chunk; the 16-byte piece p of token t is kept
    // at slot p ^ (t % 16), so the 16 lanes of a read clock (16 tokens, one piece) spread over 16 bank groups
    constexpr int TPI = 4 / XS, LPT = 64 / TPI;                 // tokens per instruction, lanes (= pieces) per token
    uint32_t xsrc;
    {
        const int rowx = wave * TPI + lane / LPT;
        const int piece = (lane % LPT) ^ (rowx & 15);
        xsrc = (uint32_t)(min(rowx, a.B - 1) * a.ldxh + piece * 8);
    }
    const bool xo = wave * TPI < 16 * NBLK;                     // this wave takes part in the x copies
    auto copy_x = [&](int c) {
        if (xo) __builtin_amdgcn_global_load_lds((gptr_t)(a.xh + c * (XS * 128) + xsrc), (lptr_t)(xs + (c & 1) * XBUF + wave * TPI * XPITCH), 16, 0, 0);
    };
    // weights: instruction n of a step fills rows 8 n .. 8 n + 7; lane i lands in row 8 n + i / 8, slot i % 8 and
    // fetches the piece the swizzle keeps there
    const int8_t* wsrc[2];
#pragma unroll
    for (int n = 0; n < 2; ++n) {
        const int rw = 8 * n + (lane >> 3);
        const int piece = (lane & 7) ^ ((rw >> 1) & 7);
        wsrc[n] = a.q + (int64_t)min(task * 16 + rw, a.V - 1) * C + piece * 16;
    }
    auto copy_w = [&](int s) {
#pragma unroll
        for (int n = 0; n < 2; ++n)
            __builtin_amdgcn_global_load_lds((gptr_t)(wsrc[n] + s * 128), (lptr_t)(wl + (s % Q8L_D) * 2048 + n * 1024), 16, 0, 0);
    };
    // scales of chunk c: lane i fetches dword i % 4 of row i / 4
    const char* ssrc = (const char*)(a.sc + (int64_t)min(task * 16 + (lane >> 2), a.V - 1) * nblk) + (lane & 3) * 4;
    auto copy_s = [&](int c) {
        __builtin_amdgcn_global_load_lds((gptr_t)(ssrc + c * 16), (lptr_t)(sl_ + (c % (D - 1)) * 256), 4, 0, 0);
    };
    const uint32_t xrow = (uint32_t)r * XPITCH, xsw = (uint32_t)r;
    const uint32_t wsw = (uint32_t)((r >> 1) & 7);
    const uint32_t w0 = (uint32_t)r * 128 + (((uint32_t)(2 * g) ^ wsw) << 4), w1 = (uint32_t)r * 128 + (((uint32_t)(2 * g + 1) ^ wsw) << 4);

    float4v acc[NBLK];
#pragma unroll
    for (int nb = 0; nb < NBLK; ++nb) acc[nb] = float4v{0.f, 0.f, 0.f, 0.f};

    // Issue order per wave (X = this wave's x copy of a chunk, S = scales of a chunk, W = the 2 copies of a step):
    // S(c) goes right before W(2c); step s starts (even s: after the wait and the barrier, then X(s/2 + 1)) with the
    // refill of step s + D - 1.  Waits count the operations that may stay in flight:
    //   even s (needs X, S, W of its chunk):  D = 3: W(s+1) -> 2;           D = 4: W(s+1) S W(s+2) -> 5
    //   odd s (needs W(s)):  D = 3: X S W(s+1) W(s+2) -> 5 + x;  D = 4: S W(s+1) X W(s+2) S W(s+3) -> 8 + x
    // and fall back to "everything" near the end of the row, where refills stop.
    auto refill = [&](int f) {
        if (f < nsteps) {
            if (!(f & 1)) copy_s(f >> 1);
            copy_w(f);
        }
    };
    copy_x(0);
#pragma unroll
    for (int t = 0; t < D - 1; ++t) refill(t);
    for (int s = 0; s < nsteps; ++s) {
        const int c = s >> 1, odd = s & 1, cx = s / XS;         // chunk of scales, step in it, chunk of x
        if (XS == 1) {
            // every step opens an x chunk: X(s) was issued one step ago, before [S] W(s + 1)
            if (s + 1 < nsteps) { if (odd) __builtin_amdgcn_s_waitcnt(q8_vmcnt(3)); else __builtin_amdgcn_s_waitcnt(q8_vmcnt(2)); }
            else __builtin_amdgcn_s_waitcnt(q8_vmcnt(0));
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
            if (cx + 1 < nchunks) copy_x(cx + 1);
            refill(s + D - 1);
        } else if (!odd) {
            if (s + D - 2 < nsteps) __builtin_amdgcn_s_waitcnt(q8_vmcnt(D == 3 ? 2 : 5));
            else __builtin_amdgcn_s_waitcnt(q8_vmcnt(0));
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
            if (cx + 1 < nchunks) copy_x(cx + 1);
            refill(s + D - 1);
        } else {
            refill(s + D - 1);
            if (s + D - 1 < nsteps) {
                if (xo) __builtin_amdgcn_s_waitcnt(q8_vmcnt(D == 3 ? 6 : 9));
                else __builtin_amdgcn_s_waitcnt(q8_vmcnt(D == 3 ? 5 : 8));
            } else {
                __builtin_amdgcn_s_waitcnt(q8_vmcnt(0));
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        const unsigned char* st = wl + (s % Q8L_D) * 2048;
        const u32x4 wq[2] = {*reinterpret_cast<const u32x4*>(st + w0), *reinterpret_cast<const u32x4*>(st + w1)};
        const half_t sh = __builtin_bit_cast(half_t, *reinterpret_cast<const uint16_t*>(sl_ + (c % (D - 1)) * 256 + r * 16 + odd * 8 + g * 2));
        const half2v s2 = {sh, sh};
        const unsigned char* xc = xs + (cx & 1) * XBUF + xrow;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            half2v p[8];
#pragma unroll
            for (int k = 0; k < 4; ++k) i8x4_to_h2(wq[j][k], p[2 * k], p[2 * k + 1]);
#pragma unroll
            for (int k = 0; k < 8; ++k) p[k] = p[k] * s2;
            half8v a0, a1;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                a0[2 * k] = p[k][0]; a0[2 * k + 1] = p[k][1];
                a1[2 * k] = p[4 + k][0]; a1[2 * k + 1] = p[4 + k][1];
            }
            const uint32_t p0 = (uint32_t)((s % XS) * 16 + (2 * g + j) * 2);   // x pieces (8 halves each) of these 16 columns
#pragma unroll
            for (int nb = 0; nb < NBLK; ++nb) {
                const unsigned char* xt = xc + nb * (16 * XPITCH);
                const half8v x0 = *reinterpret_cast<const half8v*>(xt + ((p0 ^ xsw) << 4));
                const half8v x1 = *reinterpret_cast<const half8v*>(xt + (((p0 + 1) ^ xsw) << 4));
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, x0, acc[nb], 0, 0, 0);
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, x1, acc[nb], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    if (!active) return;
    const int orow = task * 16 + g * 4;
#pragma unroll
    for (int nb = 0; nb < NBLK; ++nb) {
        const int tok = nb * 16 + r;
        if (tok >= a.B) continue;
        if (a.vec_y && a.y_dtype != SQ_F32 && orow + 4 <= a.V) {
            uint16_t o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = a.y_dtype == SQ_BF16 ? f2bf(acc[nb][e]) : f2h(acc[nb][e]);
            *reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(a.y) + (int64_t)tok * a.ldy + orow) =
                u32x2{(uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16)};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (orow + e < a.V) store_y(a.y, a.y_dtype, (int64_t)tok * a.ldy + orow + e, acc[nb][e]);
        }
    }
}

// N consecutive outputs of type T from fp32 values: 16-byte stores when the destination allows it.
template <int DT, int N>
__device__ __forceinline__ void store_run(typename store_as<DT>::type* dst, const float (&v)[N], bool vec) {
    typedef typename store_as<DT>::type T;
    if (vec) {
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int k = 0; k < N; k += 4)
                *reinterpret_cast<float4v*>(dst + k) = float4v{v[k], v[k + 1], v[k + 2], v[k + 3]};
        } else {
#pragma unroll
            for (int k = 0; k < N; k += 8) {
                u32x4 p;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    p[e] = (uint32_t)store_as<DT>::cvt(v[k + 2 * e]) | ((uint32_t)store_as<DT>::cvt(v[k + 2 * e + 1]) << 16);
                *reinterpret_cast<u32x4*>(dst + k) = p;
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < N; ++k) dst[k] = store_as<DT>::cvt(v[k]);
    }
}

// Rows [r0, r1) as dense values, one 16-byte load (16 weights, half a block) per thread.
template <int DT>
__global__ __launch_bounds__(256) void q8_dequant_kernel(const int8_t* __restrict__ q, const uint16_t* __restrict__ sc,
                                                         int C, typename store_as<DT>::type* __restrict__ out,
                                                         int64_t ld_out, int r0, int64_t n16, int vec) {
    const int per_row = C >> 4;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < n16; t += (int64_t)gridDim.x * 256) {
        const int rr = (int)(t / per_row), c = (int)(t - (int64_t)rr * per_row) * 16;
        const int64_t row = r0 + rr;
        const u32x4 v = *reinterpret_cast<const u32x4*>(q + row * C + c);
        const float s = h2f(sc[row * (C >> 5) + (c >> 5)]);
        float o[16];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t w = v[k];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[4 * k + e] = (float)(int8_t)(w >> (8 * e)) * s;
        }
        store_run<DT, 16>(out + (int64_t)rr * ld_out + c, o, vec != 0);
    }
}

// Embedding rows: one 16-byte load (32 weights, one block) per thread.  Ids outside [0, V) give a row of zeros.
template <int DT>
__global__ __launch_bounds__(256) void q4_embed_kernel(const uint8_t* __restrict__ q, const uint16_t* __restrict__ sc,
                                                       int V, int C, const int64_t* __restrict__ ids, int64_t n_ids,
                                                       typename store_as<DT>::type* __restrict__ out, int64_t ld_out, int vec) {
    typedef typename store_as<DT>::type T;
    const int nblk = C >> 5;
    const int64_t total = n_ids * nblk;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < total; t += (int64_t)gridDim.x * 256) {
        const int64_t i = t / nblk;
        const int b = (int)(t - i * nblk);
        const int64_t id = ids[i];
        T* dst = out + i * ld_out + b * 32;
        float o[32];
        if (id < 0 || id >= V) {
#pragma unroll
            for (int k = 0; k < 32; ++k) o[k] = 0.f;
        } else {
            const u32x4 v = *reinterpret_cast<const u32x4*>(q + id * (C >> 1) + b * 16);
            const float s = h2f(sc[id * nblk + b]);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t w = v[k];
#pragma unroll
                for (int e = 0; e < 8; ++e) o[8 * k + e] = (float)((int)((w >> (4 * e)) & 15u) - 8) * s;
            }
        }
        store_run<DT, 32>(dst, o, vec != 0);
    }
}

static int q8_pass_rows(int B, int C) {
    int nb = B > 2 ? 4 : B > 1 ? 2 : 1;
    while (nb > 1 && nb * C > Q8_LDS_HALVES) nb >>= 1;
    return nb;
}

// The MFMA passes need C % 256 == 0 (whole 256-column chunks of x) and 64 activation rows of C halves within
// 32-bit offsets.
static bool q8_mfma_ok(int C) { return C % 256 == 0 && (int64_t)C * 64 < ((int64_t)1 << 31); }

// from 3 rows the MFMA passes win over the 4-row kernel (152,064 x 3,584: 106 against 148 us; 248,320 x 5,120: 246
// against 255 us); 2 rows stay on the exact-product kernel (106-115 / 228 us)
bool q8_mid(int C, int B) { return B > 2 && B <= Q8_MFMA_MAX_ROWS && q8_mfma_ok(C); }
size_t q8_mid_workspace(int C, int B) { return q8_mid(C, B) ? (((size_t)B * C * 2) + 255) & ~(size_t)255 : 0; }

int launch_q8_mid(const int8_t* q, const uint16_t* sc, int V, int C, const void* x, int x_dtype, int64_t ldx, void* y,
                  int y_dtype, int64_t ldy, int B, void* ws, size_t ws_bytes, hipStream_t s) {
    if (ws_bytes < q8_mid_workspace(C, B)) return fail(SQ_EWORKSPACE, "sq_q8_linear: workspace %zu < %zu", ws_bytes, q8_mid_workspace(C, B));
    const size_t ys = y_dtype == SQ_F32 ? 4 : 2;
    // fp16 activations with 16-byte aligned rows are copied to LDS from where they are; anything else goes through
    // an fp16 copy in the workspace first
    const uint16_t* xh = (const uint16_t*)x;
    int64_t ldxh = ldx;
    int rc;
    if (x_dtype != SQ_F16 || ((uintptr_t)x & 15) || ldx % 8 || ldx * 64 >= ((int64_t)1 << 31)) {
        const int64_t n = (int64_t)B * C;
        const int64_t want = (n + 255) / 256;
        hipLaunchKernelGGL(q8_x_kernel, dim3((unsigned)(want < 4096 ? want : 4096)), dim3(256), 0, s, (const uint16_t*)x, ldx, B,
                           C, x_dtype, (uint16_t*)ws);
        rc = check_launch("q8_x_kernel");
        if (rc) return rc;
        xh = (const uint16_t*)ws;
        ldxh = C;
    }
    const int tasks = (V + 15) / 16;
    for (int b0 = 0; b0 < B;) {
        const int pass = B - b0 > 32 ? 64 : 32;                  // activation rows of this pass at most
        Q8MfmaArgs a{};
        a.q = q; a.sc = sc;
        a.xh = xh + (int64_t)b0 * ldxh;
        a.ldxh = (int)ldxh;
        a.y = (char*)y + (size_t)b0 * ldy * ys;
        a.ldy = ldy; a.V = V; a.C = C; a.B = B - b0 < pass ? B - b0 : pass; a.y_dtype = y_dtype; a.tasks = tasks;
        a.vec_y = ((uintptr_t)a.y & 7) == 0 && ldy % 4 == 0;
        static bool raised = false;
        if (!raised) {
            (void)hipFuncSetAttribute((const void*)q8_mfma_kernel<1, 8, 3, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)q8_mfma_kernel<2, 16, 3, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)q8_mfma_kernel<2, 8, 3, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute((const void*)q8_mfma_kernel<4, 16, 3, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipGetLastError();
            raised = true;
        }
        // 17-32 rows: one workgroup of 16 waves per CU sharing 256-column x chunks, unless its workgroups fill the last
        // round of the chip badly; then 8 waves with 128-column chunks (a barrier per step, two workgroups per CU).
        // Measured: 152,064 x 3,584 (594 workgroups of 16 waves, 2.3 rounds) 126 against 116 us; 248,320 x 5,120
        // (970, 3.8 rounds) 265 against 278 us.
        const int cus = device_cus(), n16 = (tasks + 15) / 16;
        const bool x128 = (double)n16 / ((double)((n16 + cus - 1) / cus) * cus) < 0.85;
        if (a.B > 32)                                           // 33-64 rows: 16 waves share 128-column chunks of 64 tokens
            hipLaunchKernelGGL((q8_mfma_kernel<4, 16, 3, 1>), dim3((unsigned)((tasks + 15) / 16)), dim3(1024), q8l_lds_bytes(4, 16, 3, 1), s, a);
        else if (a.B > 16 && x128)
            hipLaunchKernelGGL((q8_mfma_kernel<2, 8, 3, 1>), dim3((unsigned)((tasks + 7) / 8)), dim3(512), q8l_lds_bytes(2, 8, 3, 1), s, a);
        else if (a.B > 16)
            hipLaunchKernelGGL((q8_mfma_kernel<2, 16, 3, 2>), dim3((unsigned)((tasks + 15) / 16)), dim3(1024), q8l_lds_bytes(2, 16, 3, 2), s, a);
        else
            hipLaunchKernelGGL((q8_mfma_kernel<1, 8, 3, 2>), dim3((unsigned)((tasks + 7) / 8)), dim3(512), q8l_lds_bytes(1, 8, 3, 2), s, a);
        rc = check_launch("q8_mfma_kernel");
        if (rc) return rc;
        b0 += a.B;
    }
    return SQ_OK;
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
    const int64_t per16 = out_dtype == SQ_F32 ? 4 : 8;          // elements per 16 bytes
    const int vec = ((uintptr_t)out & 15) == 0 && ld_out % per16 == 0;
    if (out_dtype == SQ_F32)
        hipLaunchKernelGGL(q8_dequant_kernel<SQ_F32>, dim3(grid), dim3(256), 0, s, q, sc, C, (float*)out, ld_out, r0, n16, vec);
    else if (out_dtype == SQ_F16)
        hipLaunchKernelGGL(q8_dequant_kernel<SQ_F16>, dim3(grid), dim3(256), 0, s, q, sc, C, (uint16_t*)out, ld_out, r0, n16, vec);
    else
        hipLaunchKernelGGL(q8_dequant_kernel<SQ_BF16>, dim3(grid), dim3(256), 0, s, q, sc, C, (uint16_t*)out, ld_out, r0, n16, vec);
    return check_launch("q8_dequant_kernel");
}

int launch_q4_embed(const uint8_t* q, const uint16_t* sc, int V, int C, const int64_t* ids, int64_t n_ids, void* out,
                    int out_dtype, int64_t ld_out, hipStream_t s) {
    const int64_t total = n_ids * (C >> 5);
    if (total == 0) return SQ_OK;
    const int64_t want = (total + 255) / 256;
    const unsigned grid = (unsigned)(want < 65536 ? want : 65536);
    const int64_t per16 = out_dtype == SQ_F32 ? 4 : 8;
    const int vec = ((uintptr_t)out & 15) == 0 && ld_out % per16 == 0;
    if (out_dtype == SQ_F32)
        hipLaunchKernelGGL(q4_embed_kernel<SQ_F32>, dim3(grid), dim3(256), 0, s, q, sc, V, C, ids, n_ids, (float*)out, ld_out, vec);
    else if (out_dtype == SQ_F16)
        hipLaunchKernelGGL(q4_embed_kernel<SQ_F16>, dim3(grid), dim3(256), 0, s, q, sc, V, C, ids, n_ids, (uint16_t*)out, ld_out, vec);
    else
        hipLaunchKernelGGL(q4_embed_kernel<SQ_BF16>, dim3(grid), dim3(256), 0, s, q, sc, V, C, ids, n_ids, (uint16_t*)out, ld_out, vec);
    return check_launch("q4_embed_kernel");
}

}  // namespace sq
