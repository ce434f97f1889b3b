// bfloat16 matrix products on the matrix cores: out[M, N] = x[M, K] . w[N, K]^T, float32
// accumulation, output bfloat16 or float32.  Two kernels:
//
//  * skinny (M <= 16, decode): bound by reading w once from HBM.  A workgroup owns 16 rows of
//    w; its waves split K in interleaved blocks of 128, each wave streaming its part of the
//    rows straight from global memory into v_mfma_f32_16x16x32_bf16 operands (w is the A
//    operand, x^T the B operand); the waves' partial sums meet in LDS.  No split-K workspace,
//    no atomics: the order of the sums is fixed.
//  * tiled (M > 16): workgroup tiles of 64x128 to 256x256 by 64 (the small ones with K cut into
//    shares and a reduction kernel where whole-K tiles would leave CUs idle) that go from global
//    memory straight into a ring of LDS stages, 4 waves built from v_mfma_f32_32x32x16_bf16 in
//    a hand-scheduled loop.  Workgroups are renumbered so that each XCD's L2 sees neighbouring
//    tiles.
//
// The reference's linear kernel computes the same product with one thread per output element
// and no matrix instruction (src/kernels/linear.cu:7-56).
#include "common.h"

namespace lc {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

template <typename TO> __device__ __forceinline__ void store_out(TO* p, float v);
template <> __device__ __forceinline__ void store_out<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_out<bf16>(bf16* p, float v) { *p = static_cast<bf16>(v); }

// two adjacent elements in one store; p is aligned to the pair
template <typename TO> __device__ __forceinline__ void store_pair(TO* p, float a, float b);
template <> __device__ __forceinline__ void store_pair<float>(float* p, float a, float b) {
    *reinterpret_cast<float2*>(p) = make_float2(a, b);
}
template <> __device__ __forceinline__ void store_pair<bf16>(bf16* p, float a, float b) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 v;
    v[0] = static_cast<bf16>(a);
    v[1] = static_cast<bf16>(b);
    *reinterpret_cast<bf16x2*>(p) = v;
}

// the value of another lane of the same row of 16 lanes, by a DPP move: CTRL 0xB1 swaps
// neighbours (lane ^ 1), 0x128 rotates the row by 8 (lane ^ 8).  All lanes must be active.
template <int CTRL> __device__ __forceinline__ float lane_swap(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// silu(g) * u with silu(g) = g / (1 + exp(-g))   (reference: src/kernels/swiglu.cu:8,31-35).
// exp and the reciprocal are the hardware's single instructions (about one unit in the last
// place each); the results of these products are rounded to bfloat16 afterwards.
__device__ __forceinline__ float swiglu_f(float g, float u) {
    return g * __builtin_amdgcn_rcpf(1.f + __expf(-g)) * u;
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) const void* glb_ptr_t;

// ------------------------------------------------------------------------------- skinny
constexpr int SK_KBLOCK = 128; // k elements per wave iteration

// What a skinny product can take over from the norm kernels around it (decode steps are
// bound by the number of kernels they start, not by the work of the small ones):
//   SCALE (with epilogue 0 or 1): x holds rows h * norm_weight that still lack their common
//     factor rsqrt(mean(h^2) + eps); scale_partials [scale_count][stride] holds pieces of every
//     row's sum of squares (row m at [piece][m]; stride: M rounded up to a power of two, so
//     that every workgroup reads no more of them than it must); the factor is applied to the
//     float32 sums.
//   epilogue 2: resid [M, N] is the float32 residual stream: resid += x . w^T in place; the
//     kernel also leaves next_x = bf16(resid * next_w) and, per workgroup, the sums of squares
//     of its columns of the new rows in next_partials [gridDim.x][stride]: what a SCALE product
//     (or rmsnorm) needs to go on without a norm kernel in between.
struct SkinnyFuse {
    const float* scale_partials;
    int scale_count;
    float scale_eps;
    float* resid;
    const float* next_w;
    bf16* next_x;
    float* next_partials;
    int stride;
};
constexpr int SK_MAX_PIECES = 512;   // pieces of a sum of squares that a SCALE product reads

// the k blocks of one tile's rows of w that a wave works on (a block past the end is loaded, not used)
template <int XR, int WAVES>
__device__ __forceinline__ void load_w_blocks(bf16x8 (&a)[XR][4], const bf16* wp, int wave, int kblocks) {
#pragma unroll
    for (int i = 0; i < XR; ++i) {
        const int kb = min(wave + i * WAVES, kblocks - 1);
#pragma unroll
        for (int j = 0; j < 4; ++j) a[i][j] = *reinterpret_cast<const bf16x8*>(wp + kb * SK_KBLOCK + j * 32);
    }
}

// MT: tiles of 16 rows of x; NT: tiles of 16 rows of w per workgroup tile; the WAVES waves of a
// workgroup take the k blocks in turn.  A workgroup takes the tiles blockIdx.x, blockIdx.x +
// gridDim.x, ...  XR = 0: one tile per workgroup is the intended use, and x is read as it is
// needed.  XR > 0 (K <= XR * WAVES * 128): every wave keeps the part of x that its k blocks
// need in registers for all of its workgroup's tiles.  Every workgroup has to fetch x through
// its CU's path from L2, which is what bounds this kernel from a few rows of x on: with three
// tiles per workgroup, x costs a third.
template <int MT, int NT, int WAVES, int UNROLL, int EPI, bool SCALE, int XR, typename TO>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16* __restrict__ x,
                                                                 const bf16* __restrict__ w,
                                                                 TO* __restrict__ out, int M, int N,
                                                                 int K, int rows, SkinnyFuse fuse) {
    static_assert(WAVES == 16, "the epilogues lay 1024 threads over a workgroup's results");
    static_assert(MT == 1, "up to 16 rows of x");
    static_assert(!(SCALE && EPI == 2), "both would use the same words of LDS");
    static_assert(XR == 0 || NT == 1, "x stays in registers for single tiles only");
    // a wave's sums of one tile take RS floats: 256 and a pad that puts the four quarters of
    // the waves, which the epilogue's lanes read side by side, on different banks
    constexpr int RS = 256 + 4;
    __shared__ float red[WAVES * NT * RS];
    __shared__ float pieces[WAVES][16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    // a work item ("tile" below) is `rows` <= 16 NT rows of w; with fewer than 16 NT the last of
    // its blocks of 16 is partly idle, which costs nothing here (the kernel waits for memory) and
    // lets the host cut N into as many equal items as fill the CUs evenly
    const int tiles = (N + rows - 1) / rows;
    const int kblocks = K / SK_KBLOCK;

    // loads whose values are wanted only after the products; issued first, they are back
    // before the first operand is
    float piece[SK_MAX_PIECES / 64];
    if (SCALE) {
#pragma unroll
        for (int i = 0; i < SK_MAX_PIECES / 64; ++i) {   // thread t: row t % stride of pieces t / stride + ...
            const int at = threadIdx.x + WAVES * 64 * i;
            piece[i] = at < fuse.scale_count * fuse.stride ? fuse.scale_partials[at] : 0.f;
        }
    }
    // the rows' sums of squares go through LDS: each wave leaves its pieces' sums there ...
    auto leave_pieces = [&]() {
        float sum = 0.f;       // the lanes l with l % stride = m hold row m
#pragma unroll
        for (int i = 0; i < SK_MAX_PIECES / 64; ++i) sum += piece[i];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1)
            if (off >= fuse.stride) sum += __shfl_xor(sum, off, 64);
        if (lane < fuse.stride) pieces[wave][lane] = sum;
    };
    // ... and, after a barrier, every lane gets the factor of row r
    auto row_factor = [&]() {
        float ss = 0.f;
        if (r < fuse.stride) {
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) ss += pieces[wv][r];
        }
        return rsqrtf(ss / (float)K + fuse.scale_eps);
    };
    float factor = 1.f;
    const bf16* xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xp[mt] = x + (size_t)min(mt * 16 + r, M - 1) * K + g * 8;
    bf16x8 xb[XR > 0 ? XR : 1][4];
    if (XR > 0) {
#pragma unroll
        for (int i = 0; i < XR; ++i) {
            const int kb = min(wave + i * WAVES, kblocks - 1);   // a block past the end is loaded, not used
#pragma unroll
            for (int j = 0; j < 4; ++j) xb[i][j] = *reinterpret_cast<const bf16x8*>(xp[0] + kb * SK_KBLOCK + j * 32);
        }
    }

    // XR of 1 or 2: registers are left for the next tile's part of w as well
    constexpr bool AHEAD = XR == 1 || XR == 2;
    bf16x8 a_now[XR > 0 ? XR : 1][4], a_next[XR > 0 ? XR : 1][4];
    bool first = true;
    // one tile: its rows of w are in a_use (XR > 0 with AHEAD) or loaded here; a_fill takes the next tile's
    auto one_tile = [&](const int tile, bf16x8 (&a_use)[XR > 0 ? XR : 1][4], bf16x8 (&a_fill)[XR > 0 ? XR : 1][4]) {
        const int n0 = tile * rows, n_end = min(N, n0 + rows);
        // The epilogue's layout: wave q and lane (row m = lane % 16, quarter = lane / 16) add up,
        // over the waves 4 quarter .. 4 quarter + 3, the sums for row m and column
        // n0 + 16 nt + 4 (q % 4) + q / 4; the quarters then meet by two lane exchanges, and the
        // lanes of quarter 0 own the result.
        const int e_n = n0 + (wave & 3) * 4 + (wave >> 2);
        float e_resid[NT], e_w[NT];
        if (EPI == 2) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const bool mine = g == 0 && r < M && e_n + nt * 16 < n_end;
                e_resid[nt] = mine ? fuse.resid[(size_t)r * N + e_n + nt * 16] : 0.f;
                e_w[nt] = mine ? fuse.next_w[e_n + nt * 16] : 0.f;
            }
        }

        const bf16* wp[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) wp[nt] = w + (size_t)min(n0 + nt * 16 + r, n_end - 1) * K + g * 8;

        floatx4 acc[NT][MT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

        if constexpr (XR > 0) {
            if (!AHEAD) load_w_blocks<XR, WAVES>(a_use, wp[0], wave, kblocks);
            if (AHEAD && tile + gridDim.x < tiles) {
                // the next tile's rows of w are on their way while this tile's sums meet in LDS
                const int n_next = (tile + gridDim.x) * rows;
                load_w_blocks<XR, WAVES>(a_fill, w + (size_t)min(n_next + r, min(N, n_next + rows) - 1) * K + g * 8, wave, kblocks);
            }
#pragma unroll
            for (int i = 0; i < XR; ++i) {
                if (wave + i * WAVES < kblocks) {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[0][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_use[i][j], xb[i][j], acc[0][0], 0, 0, 0);
                }
            }
        } else {
#pragma unroll UNROLL
            for (int kb = wave; kb < kblocks; kb += WAVES) {
                const int k0 = kb * SK_KBLOCK;
                bf16x8 a[NT][4];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int j = 0; j < 4; ++j) a[nt][j] = *reinterpret_cast<const bf16x8*>(wp[nt] + k0 + j * 32);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    bf16x8 b[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) b[j] = *reinterpret_cast<const bf16x8*>(xp[mt] + k0 + j * 32);
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt][j], b[j], acc[nt][mt], 0, 0, 0);
                }
            }
        }
        // acc[nt][0][v] = partial out[m = lane%16][n = n0 + nt*16 + (lane/16)*4 + v], kept at [v * 64 + lane]
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[(wave * NT + nt) * RS + v * 64 + lane] = acc[nt][0][v];
        if (SCALE && XR == 0 && first) leave_pieces();
        first = false;
        __syncthreads();
        // element e of a tile's 256 sums, over all waves (every lane of the four quarters gets it)
        auto total_of = [&](int nt, int e) {
            float t = 0.f;
#pragma unroll
            for (int k = 0; k < 4; ++k) t += red[((g * 4 + k) * NT + nt) * RS + e];
            t += __shfl_xor(t, 16, 64);
            t += __shfl_xor(t, 32, 64);
            return t;
        };
        const int e_mine = wave * 16 + r;     // = v * 64 + (lane of the product) with v = wave / 4
        if (EPI == 2) {
            float sq = 0.f;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const float t = total_of(nt, e_mine);
                if (g == 0 && r < M && e_n + nt * 16 < n_end) {
                    const float v = e_resid[nt] + t;
                    fuse.resid[(size_t)r * N + e_n + nt * 16] = v;
                    fuse.next_x[(size_t)r * N + e_n + nt * 16] = static_cast<bf16>(v * e_w[nt]);
                    sq += v * v;
                }
            }
            // a row's squares: every wave holds one column of each of the tile's blocks of 16
            if (g == 0) pieces[wave][r] = sq;
            __syncthreads();
            if (threadIdx.x < fuse.stride) {
                float row = 0.f;
#pragma unroll
                for (int wv = 0; wv < WAVES; ++wv) row += pieces[wv][threadIdx.x];
                fuse.next_partials[(size_t)tile * fuse.stride + threadIdx.x] = row;
            }
        } else {
            if (SCALE && XR == 0) factor = row_factor();
            if (EPI == 0) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const float t = total_of(nt, e_mine);
                    const int n = e_n + nt * 16;
                    if (g == 0 && r < M && n < n_end) store_out<TO>(out + (size_t)r * N + n, t * factor);
                }
            } else {
                // rows of w come in blocks of 16: 8 gate rows, then their 8 up rows; out has N / 2
                // columns.  The waves with q % 4 < 2 hold gate rows; the up row of each is two
                // waves (32 elements) further on.
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    if ((wave & 3) < 2) {
                        const float gate = total_of(nt, e_mine), up = total_of(nt, e_mine + 32);
                        const int n = e_n + nt * 16;
                        const int col = (n >> 4) * 8 + (n & 7);
                        if (g == 0 && r < M && n < n_end)
                            store_out<TO>(out + (size_t)r * (N / 2) + col, swiglu_f(gate * factor, up * factor));
                    }
                }
            }
        }
        if (tile + gridDim.x < tiles) __syncthreads();   // red and pieces are written again
    };
    if constexpr (AHEAD) {
        // two sets of registers take turns, so that no value has to be moved (a move would
        // wait for the loads that are meant to stay in flight)
        int tile = blockIdx.x;
        if (tile < tiles)
            load_w_blocks<XR, WAVES>(a_now, w + (size_t)min(tile * rows + r, min(N, (tile + 1) * rows) - 1) * K + g * 8, wave, kblocks);
        if (SCALE) {   // a workgroup of many tiles waits for the pieces once, while x and the first tile's rows of w are on their way
            leave_pieces();
            __syncthreads();
            factor = row_factor();
        }
        while (tile < tiles) {
            one_tile(tile, a_now, a_next);
            tile += gridDim.x;
            if (tile >= tiles) break;
            one_tile(tile, a_next, a_now);
            tile += gridDim.x;
        }
    } else {
        if (SCALE && XR > 0) {
            leave_pieces();
            __syncthreads();
            factor = row_factor();
        }
        for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x) one_tile(tile, a_now, a_now);
    }
}

// ------------------------------------------------------------------------------- skinny, rows in runs
// The same product (up to 16 rows of x, tiles of up to 16 rows of w, the same epilogues), with
// w read as memory likes it.  The matrix-core operand of the kernel above makes every load
// instruction fetch 64 bytes of each of 16 rows of w, which are K elements apart: measured,
// such loads move 4.2 to 4.4 TB/s where loads of 1 KB runs move 5.4 to 6.0.  Here a wave's load
// instruction takes 1 KB of ONE row (512 k) straight into LDS (global_load_lds_dwordx4), the 16
// waves of a workgroup fill one stage (16 rows x 512 k) of a ring of eight, and the operands
// are read from LDS: wave q multiplies the k-step q of every stage (32 k, one product), so a
// wave needs of x only its own K / 16 columns, which it keeps in registers.  Within a row the
// 16-byte chunk c lies at place c ^ row: the 16 lanes that LDS serves together (16 rows, one
// chunk) then use all banks.  The ring runs on across the workgroup's tiles; a stage is
// reused one barrier after its last reader.  Counted waits and raw barriers: the compiler
// would wait for all loads in flight at every LDS access and barrier.
constexpr int SR_K = 512;             // k elements of a run
constexpr int SR_RING = 8;
constexpr int SR_STAGE = 16 * SR_K;   // bf16 elements of a stage

__device__ __forceinline__ void lds_put(unsigned addr, float v) {
    asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(v) : "memory");
}
__device__ __forceinline__ float lds_get(unsigned addr) {
    float v;
    asm volatile("ds_read_b32 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
}

// at most min(n, MAXN) of the youngest loads may still be in flight
template <int MAXN> __device__ __forceinline__ void wait_vmcnt_upto(int n) {
    static_assert(MAXN == 6 || MAXN == 12, "the cases below");
    if (n >= MAXN) { wait_vmcnt<MAXN>(); return; }
    if (MAXN == 12) n >>= 1;      // even numbers only: two loads a stage
    switch (n) {
    case 0: wait_vmcnt<0>(); break;
    case 1: wait_vmcnt<MAXN / 6>(); break;
    case 2: wait_vmcnt<2 * (MAXN / 6)>(); break;
    case 3: wait_vmcnt<3 * (MAXN / 6)>(); break;
    case 4: wait_vmcnt<4 * (MAXN / 6)>(); break;
    default: wait_vmcnt<5 * (MAXN / 6)>(); break;
    }
}
// a barrier for LDS written by ordinary stores (it does not wait for global loads in flight)
__device__ __forceinline__ void raw_barrier() {
    // one statement: the compiler keeps ordinary stores before it, and the wait cannot part from the barrier
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory");
}

// XS > 0 (K <= XS * 512): a wave keeps its columns of x in registers for all of its workgroup's
// tiles.  XS = 0 (any K): a wave's 16 bytes of x for a stage travel with the stage's run of w,
// seven stages ahead, into a ring of registers.  Those loads are inline assembly (the compiler
// would wait for them, and with them for every load of the ring issued before them, at their
// first use); a register of the ring is written by the hardware long after the statement that
// names it, which is safe only because every such register is read again after the counted wait
// and before anything else may be put into it: a load whose value nobody reads would leave its
// registers to the compiler's next use while the value is still on its way.
template <int EPI, bool SCALE, int XS, typename TO>
__global__ __launch_bounds__(1024) void gemm_runs_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w,
                                                         TO* __restrict__ out, int M, int N, int K, int rows,
                                                         SkinnyFuse fuse) {
    constexpr int RS = 256 + 4;        // a wave's 256 sums, padded
    constexpr int PER = XS > 0 ? 1 : 2;   // loads a wave issues per stage
    __shared__ __attribute__((aligned(1024))) bf16 ring[SR_RING * SR_STAGE];
    __shared__ float red[16 * RS];
    __shared__ float part_sq[16][16];
    __shared__ float factors[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int tiles = (N + rows - 1) / rows;
    if ((int)blockIdx.x >= tiles) return;
    const int spt = K / SR_K;                                        // stages per tile
    const int my_tiles = (tiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    const int total_stages = my_tiles * spt;
    const unsigned ring0 = (unsigned)(uintptr_t)(lds_ptr_t)ring;
    const unsigned red0 = (unsigned)(uintptr_t)(lds_ptr_t)red;

    // this wave's columns of x: of every stage the k-step `wave`
    const bf16* xp = x + (size_t)min(r, M - 1) * K + wave * 32 + g * 8;
    bf16x8 xr[XS > 0 ? XS : SR_RING];
    if (XS > 0) {
#pragma unroll
        for (int s = 0; s < XS; ++s) xr[s] = *reinterpret_cast<const bf16x8*>(xp + min(s, spt - 1) * SR_K);
    }
    float piece[SK_MAX_PIECES / 64];
    if (SCALE) {
#pragma unroll
        for (int i = 0; i < SK_MAX_PIECES / 64; ++i) {   // thread t: row t % stride of pieces t / stride + ...
            const int at = threadIdx.x + 1024 * i;
            piece[i] = at < fuse.scale_count * fuse.stride ? fuse.scale_partials[at] : 0.f;
        }
    }

    // the loads of the ring, in the order of the stages: wave q fetches row q of the stage's tile
    int issue_tile = blockIdx.x, issue_s = 0, issued = 0;
    auto issue = [&](bf16x8& x_to) {
        const int n0 = issue_tile * rows, n_end = min(N, n0 + rows);
        const int row = min(n0 + wave, n_end - 1);
        const bf16* src = w + (size_t)row * K + issue_s * SR_K + ((lane ^ wave) * 8);
        __builtin_amdgcn_global_load_lds((glb_ptr_t)src,
            (lds_ptr_t)(ring + (issued & (SR_RING - 1)) * SR_STAGE + wave * SR_K), 16, 0, 0);
        if (XS == 0) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(x_to) : "v"(xp + issue_s * SR_K) : "memory");
        ++issued;
        if (++issue_s == spt) { issue_s = 0; issue_tile += gridDim.x; }
    };
#pragma unroll
    for (int i = 0; i < SR_RING - 1; ++i)
        if (issued < total_stages) issue(xr[XS > 0 ? 0 : i]);

    float factor = 1.f;                  // of the row that this thread's results belong to (m = thread / 16)
    if (SCALE) {
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < SK_MAX_PIECES / 64; ++i) sum += piece[i];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1)
            if (off >= fuse.stride) sum += __shfl_xor(sum, off, 64);
        if (lane < fuse.stride) part_sq[wave][lane] = sum;
        raw_barrier();
        if (threadIdx.x < 16) {
            float ss = 0.f;
            if ((int)threadIdx.x < fuse.stride)
#pragma unroll
                for (int wv = 0; wv < 16; ++wv) ss += part_sq[wv][threadIdx.x];
            factors[threadIdx.x] = rsqrtf(ss / (float)K + fuse.scale_eps);
        }
        raw_barrier();
        factor = factors[(threadIdx.x >> 4) & 15];
    }

    // the operand of this lane in a stage: row r, chunk 4 wave + g, at place chunk ^ r
    const unsigned a_at = ring0 + (r * SR_K + (((wave * 4 + g) ^ r) * 8)) * 2;
    // a thread of the first four waves owns the result (row e_m of x, row e_j of the tile)
    const int e_m = (threadIdx.x >> 4) & 15, e_j = threadIdx.x & 15;
    int stage_at = 0;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    float e_resid = 0.f, e_w = 0.f;
    auto begin_tile = [&](int tile) {
        const int n0 = tile * rows, n_end = min(N, n0 + rows);
        acc = floatx4{0.f, 0.f, 0.f, 0.f};
        if (EPI == 2 && threadIdx.x < 256 && e_m < M && n0 + e_j < n_end) {
            e_resid = fuse.resid[(size_t)e_m * N + n0 + e_j];
            e_w = fuse.next_w[n0 + e_j];
        }
    };
    // one stage: x_use holds this wave's x of the stage; the load of the stage seven on brings its x to x_fill
    auto stage = [&](const bf16x8& x_use, bf16x8& x_fill) {
        wait_vmcnt_upto<PER * (SR_RING - 2)>(PER * (issued - stage_at - 1));   // this wave's loads of the stage have landed
        __builtin_amdgcn_s_barrier();         // everybody's have; nobody reads the stage before any more
        __builtin_amdgcn_sched_barrier(0);
        bf16x8 b = x_use;
        if (XS == 0) asm volatile("" : "+v"(b));
        if (issued < total_stages) issue(x_fill);   // into the stage before
        bf16x8 a;
        asm volatile("ds_read_b128 %0, %1" : "=v"(a) : "v"(a_at + (stage_at & (SR_RING - 1)) * (SR_STAGE * 2)));
        wait_lgkmcnt<0>();
        asm volatile("" : "+v"(a));
        __builtin_amdgcn_sched_barrier(0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
        ++stage_at;
    };
    auto end_tile = [&](int tile) {
        const int n0 = tile * rows, n_end = min(N, n0 + rows);
        // acc[v] = this wave's part of out[m = lane % 16][n = n0 + 4 (lane / 16) + v]; kept at red[wave][16 m + n - n0].
        // The stores are inline assembly, where the compiler does not see that they read what the last product
        // writes: the wait states between a matrix-core write and an LDS read of the same registers (up to 19).
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_nop 15\n\ts_nop 3");
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int v = 0; v < 4; ++v) lds_put(red0 + (wave * RS + r * 16 + g * 4 + v) * 4, acc[v]);
        wait_lgkmcnt<0>();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if (threadIdx.x < 256) {
            // the sum over the waves of this thread's element, and for SwiGLU of the up row eight further on
            auto sum_of = [&](int e) {
                float t = 0.f;
#pragma unroll
                for (int w0 = 0; w0 < 16; w0 += 4) {
                    float got[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) got[k] = lds_get(red0 + ((w0 + k) * RS + e) * 4);
                    wait_lgkmcnt<0>();
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        asm volatile("" : "+v"(got[k]));
                        t += got[k];
                    }
                }
                return t;
            };
            const float t = sum_of(threadIdx.x);
            float t_up = 0.f;
            if (EPI == 1) t_up = sum_of(threadIdx.x | 8);
            const int n = n0 + e_j;
            const bool mine = e_m < M && n < n_end;
            if (EPI == 0) {
                if (mine) store_out<TO>(out + (size_t)e_m * N + n, t * factor);
            } else if (EPI == 1) {
                // rows of w come in blocks of 16: 8 gate rows, then their 8 up rows; out has N / 2 columns
                if (mine && e_j < 8)
                    store_out<TO>(out + (size_t)e_m * (N / 2) + (n >> 4) * 8 + (n & 7), swiglu_f(t * factor, t_up * factor));
            } else {
                float sq = 0.f;
                if (mine) {
                    const float v = e_resid + t;
                    fuse.resid[(size_t)e_m * N + n] = v;
                    fuse.next_x[(size_t)e_m * N + n] = static_cast<bf16>(v * e_w);
                    sq = v * v;
                }
                // a row's squares over the tile's columns: the 16 neighbouring lanes of a row of lanes
                sq += lane_swap<0xB1>(sq);                                   // lane ^ 1
                sq += lane_swap<0x4E>(sq);                                   // lane ^ 2
                sq += __shfl_xor(sq, 4, 64);
                sq += __shfl_xor(sq, 8, 64);
                if (e_j == 0 && e_m < fuse.stride) fuse.next_partials[(size_t)tile * fuse.stride + e_m] = sq;
            }
        }
        // red is written again after the next tile's stages, each of which has a barrier of its own
    };

    if constexpr (XS > 0) {
        for (int ti = 0; ti < my_tiles; ++ti) {
            const int tile = blockIdx.x + ti * gridDim.x;
            begin_tile(tile);
#pragma unroll
            for (int s = 0; s < XS; ++s)
                if (s < spt) stage(xr[s], xr[s]);
            end_tile(tile);
        }
    } else {
        // the ring of x is indexed by the stage's number among all of the workgroup's: eight at a time
        int tile = blockIdx.x, s_in = 0;
        begin_tile(tile);
        for (int st0 = 0; st0 < total_stages; st0 += SR_RING) {
#pragma unroll
            for (int k = 0; k < SR_RING; ++k) {
                if (st0 + k < total_stages) {
                    stage(xr[k], xr[(k + SR_RING - 1) % SR_RING]);
                    if (++s_in == spt) {
                        end_tile(tile);
                        s_in = 0;
                        tile += gridDim.x;
                        if (st0 + k + 1 < total_stages) begin_tile(tile);
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------- tiled
// Workgroup tile BM x BN x 64, four waves in a 2 x 2 grid, each owning (BM/64) x (BN/64) tiles
// of 32 x 32.
//
// Operand tiles go from global memory straight into LDS (global_load_lds_dwordx4: lane l's 16
// bytes land at the instruction's LDS base + 16 l, no registers in between) into a ring of
// TL_STAGES stages.  Inside a stage a row's eight 16-byte chunks are stored at column
// (chunk ^ ((row >> 1) & 7)): the 16 lanes that the LDS serves per cycle for a 128-bit read
// (16 consecutive rows, one chunk) then cover all 64 banks.
//
// The loop is scheduled by hand, because a SIMD holds a single wave of this kernel and nothing
// else hides a stall.  Per k-step of 16 the wave issues its (BM/64)*(BN/64) products; between
// them, one at a time, go the LDS reads of the NEXT k-step's operands (ds_read_b128 in inline
// assembly with explicit waits: the compiler cannot tell the stages apart and would make every
// load in flight land before any read) and, in a block's first k-step, the global loads of the
// block TL_STAGES-1 ahead.  In a block's last k-step the wave waits for its own loads of the
// next block, meets the others at a bare barrier (all waves' loads are then visible, and all
// have finished reading the stage that the next loads overwrite) and reads the next block's
// first operands while the rest of its products run.  sched_barrier pins that order.
constexpr int TL_K = 64;

// The grid's workgroups take the tiles [tile_base, tile_base + tile_count) of the tiles_m x
// tiles_n tiles of the product.
// SPLIT: blockIdx.y owns a share of the k-blocks and writes its float32 partial sums for a
// reduction kernel to add in a fixed order: to part[blockIdx.y][M][N] (splitk_reduce_kernel),
// or, if `compact`, tile by tile to part[blockIdx.y][tile - tile_base][BM][BN]
// (tail_reduce_kernel).
template <int BM, int BN, int TL_STAGES, int EPI, bool SPLIT, typename TO, int WM = 2, int WN = 2>
__global__ __launch_bounds__(64 * WM * WN) void gemm_tiled_kernel(const bf16* __restrict__ x,
                                                         const bf16* __restrict__ w,
                                                         TO* __restrict__ out, float* __restrict__ part,
                                                         int M, int N, int K, int tiles_m, int tile_base,
                                                         int tile_count, int compact, int skew_step) {
    // WM x WN waves, each owning (BM / WM) x (BN / WN) of the tile as TM x TN products of 32 x 32
    constexpr int S = TL_STAGES;
    constexpr int NW = WM * WN;
    constexpr int TM = BM / (32 * WM), TN = BN / (32 * WN);
    constexpr int KS = TL_K / 16;                             // k-steps per block
    constexpr int LPA = BM * 8 / (64 * NW), LPB = BN * 8 / (64 * NW), LP = LPA + LPB;   // load instructions per thread and stage
    static_assert(BM % (32 * WM) == 0 && BN % (32 * WN) == 0, "whole products per wave");
    static_assert((BM * 8) % (64 * NW) == 0 && (BN * 8) % (64 * NW) == 0, "whole load instructions per wave");
    constexpr int NM = TM * TN, NR = TM + TN;                 // products and operand reads per k-step
    constexpr int A_STAGE = BM * TL_K * 2, B_STAGE = BN * TL_K * 2;          // bytes
    static_assert(S >= 2 && (S == 2 ? 2 : S - 1) * LP <= 63, "the load counter holds 63");
    static_assert(S * (A_STAGE + B_STAGE) <= 160 * 1024, "LDS");
    __shared__ __attribute__((aligned(1024))) char lds[S * (A_STAGE + B_STAGE)];   // A stages, then B stages

    // renumber: workgroups go round-robin over 8 XCDs; give each XCD a contiguous run of
    // tiles, m fastest, so that one XCD's L2 keeps the w tile that its workgroups share
    const int total = tile_count;
    int id = blockIdx.x;
    {
        const int q = total >> 3, rem = total & 7;
        const int xcd = id & 7, local = id >> 3;
        id = xcd * q + min(xcd, rem) + local;   // a bijection of [0, total) for any total
    }
    const int local_tile = id;
    id += tile_base;
    const int tm = id % tiles_m, tn = id / tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = (wave / WN) * (BM / WM), wn = (wave % WN) * (BN / WN);
    const int lr = lane & 31, kg = lane >> 5;
    auto swz = [](int row) { return (row >> 1) & 7; };

    const int nk_all = K / TL_K;
    const int kb0 = SPLIT ? (int)((long long)blockIdx.y * nk_all / gridDim.y) : 0;
    const int nk = (SPLIT ? (int)((long long)(blockIdx.y + 1) * nk_all / gridDim.y) : nk_all) - kb0;

    // chunk p = (i * NW + wave) * 64 + lane of a stage holds row p / 8, global chunk (p % 8) ^ swz(row)
    const bf16* xg[LPA];
    const bf16* wg[LPB];
#pragma unroll
    for (int i = 0; i < LPA; ++i) {
        const int p = (i * NW + wave) * 64 + lane, row = p >> 3, kc = (p & 7) ^ swz(row);
        xg[i] = x + (size_t)min(m0 + row, M - 1) * K + (size_t)kb0 * TL_K + kc * 8;
    }
#pragma unroll
    for (int i = 0; i < LPB; ++i) {
        const int p = (i * NW + wave) * 64 + lane, row = p >> 3, kc = (p & 7) ^ swz(row);
        wg[i] = w + (size_t)min(n0 + row, N - 1) * K + (size_t)kb0 * TL_K + kc * 8;
    }
    // With a single row of tiles (M <= BM: decode steps of 17 to 64 tokens) every workgroup
    // streams rows of w that nobody else reads, all rows 2 K bytes apart, and all workgroups
    // would walk k in step: at any moment the whole GPU would ask for the same few columns, which
    // lie in the same memory channels (measured with rows padded by 128 bytes instead: 64 x 24576
    // x 4096 takes 37.6 instead of 46.9 us).  So each workgroup starts at a k-block of its own
    // (tile number times skew_step, modulo the number of k-blocks) and wraps around: 37.2 us.  (With several rows of tiles the workgroups that share a tile of w
    // should read it at the same time, and do.)
    const int skew = (!SPLIT && tiles_m == 1 && skew_step) ? (int)(((unsigned)id * (unsigned)skew_step) % (unsigned)nk) : 0;
    // load instruction idx (x first, then w) of block kb into a stage
    auto issue_one = [&](int idx, int kb, int stage) {
        kb += skew;
        kb -= kb >= nk ? nk : 0;
        if (idx < LPA)
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(xg[idx] + kb * TL_K),
                (lds_ptr_t)(lds + stage * A_STAGE + (idx * NW + wave) * 1024), 16, 0, 0);
        else
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(wg[idx - LPA] + kb * TL_K),
                (lds_ptr_t)(lds + S * A_STAGE + stage * B_STAGE + ((idx - LPA) * NW + wave) * 1024), 16, 0, 0);
    };
    // With two stages, a block's loads are issued a block early: in the last k-step of block it,
    // once every wave has read the last of the stage, block it + 2 goes into it, behind block
    // it + 1 that is still arriving.  (Issued only after block it + 1 has landed, the loads
    // would start with nothing in flight: their first data would be a whole latency away, and
    // the way from L2 into the CU, which bounds these kernels, would stand idle meanwhile.)
    constexpr bool EARLY = S == 2;
    constexpr int AHEAD = EARLY ? 2 : S - 1;                  // blocks in flight at the start
#pragma unroll
    for (int s = 0; s < AHEAD; ++s)
        if (s < nk) {
#pragma unroll
            for (int i = 0; i < LP; ++i) issue_one(i, s, s);
        }

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // LDS address of this lane's operand rows in stage 0, with the lane's part of the swizzle;
    // k-step ks flips chunk bits: ((2 ks + kg) ^ swz) * 16 = ((kg ^ swz) * 16) ^ (ks * 32)
    const unsigned lds0 = (unsigned)(uintptr_t)(lds_ptr_t)lds;
    unsigned pa[TM], pb[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int row = wm + i * 32 + lr;
        pa[i] = lds0 + row * 128 + ((kg ^ swz(row)) * 16);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int row = wn + j * 32 + lr;
        pb[j] = lds0 + S * A_STAGE + row * 128 + ((kg ^ swz(row)) * 16);
    }

    bf16x8 a[2][TM], b[2][TN];
    auto read_one = [&](int r, int stage, int ks, int buf) {
        if (r < TM) {
            const unsigned addr = (pa[r] ^ (ks * 32)) + stage * A_STAGE;
            asm volatile("ds_read_b128 %0, %1" : "=v"(a[buf][r]) : "v"(addr));
        } else {
            const unsigned addr = (pb[r - TM] ^ (ks * 32)) + stage * B_STAGE;
            asm volatile("ds_read_b128 %0, %1" : "=v"(b[buf][r - TM]) : "v"(addr));
        }
    };
    // the products that follow a wait must not be moved above it: tie their operands to that point
    auto tie = [&](int buf) {
#pragma unroll
        for (int i = 0; i < TM; ++i) asm volatile("" : "+v"(a[buf][i]));
#pragma unroll
        for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(b[buf][j]));
    };
    auto product = [&](int k, int buf) {
        const int i = k / TN, j = k % TN;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[buf][i], b[buf][j], acc[i][j], 0, 0, 0);
    };

    // where the reads and loads sit among the NM products of a k-step
    constexpr int QR = (2 * NR + NM - 1) / NM;                 // reads after each product, from the first on
    constexpr int RS = (NR + QR - 1) / QR;                     // products that the reads take
    constexpr int QL = NM > RS ? (LP + (NM - RS) - 1) / (NM - RS) : LP;   // loads after each later product
    constexpr int BAR = NM / 4;                                // the product after which a block's last k-step syncs
    constexpr int QT = NM - BAR - 1 > 0 ? (NR + (NM - BAR - 1) - 1) / (NM - BAR - 1) : NR;

    // block 0 has landed when at most the younger blocks are still in flight
    if (nk >= AHEAD) wait_vmcnt<(AHEAD - 1) * LP>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int r = 0; r < NR; ++r) read_one(r, 0, 0, 0);

    int stage = 0, lstage = S - 1;   // the stage of block `it`; the stage that block it+S-1 goes to
    auto block = [&](int it, auto load_tag) {
        constexpr bool LOAD = decltype(load_tag)::value;       // block it+S-1 exists and is loaded here
        const int nstage = stage + 1 == S ? 0 : stage + 1;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int cur = ks & 1, nxt = cur ^ 1;
            wait_lgkmcnt<0>();
            tie(cur);
            __builtin_amdgcn_sched_barrier(0);
            if (ks < KS - 1) {
#pragma unroll
                for (int k = 0; k < NM; ++k) {
                    product(k, cur);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int r = k * QR; r < (k + 1) * QR; ++r)
                        if (r < NR) read_one(r, stage, ks + 1, nxt);
                    if (LOAD && !EARLY && ks == 0 && (k >= RS || NM == RS)) {
                        const int first = NM == RS ? k * QL : (k - RS) * QL;
#pragma unroll
                        for (int l = first; l < first + QL; ++l)
                            if (l < LP) issue_one(l, it + S - 1, lstage);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll
                for (int k = 0; k < NM; ++k) {
                    product(k, cur);
                    __builtin_amdgcn_sched_barrier(0);
                    if (LOAD) {
                        if (k == BAR && EARLY) {
                            __builtin_amdgcn_s_barrier();          // nobody reads this stage any more
#pragma unroll
                            for (int l = 0; l < LP; ++l) issue_one(l, it + 2, stage);
                            wait_vmcnt<LP>();                      // block it + 1 has landed
                            __builtin_amdgcn_s_barrier();
                        } else if (k == BAR) {
                            wait_vmcnt<(S - 2) * LP>();
                            __builtin_amdgcn_s_barrier();
                        }
                        if (NM - BAR - 1 > 0) {
#pragma unroll
                            for (int r = (k - BAR - 1) * QT; r < (k - BAR) * QT; ++r)
                                if (k > BAR && r < NR) read_one(r, nstage, 0, nxt);
                        } else if (k == BAR) {
#pragma unroll
                            for (int r = 0; r < NR; ++r) read_one(r, nstage, 0, nxt);
                        }
                    } else if (k == BAR) {
                        if (it + 1 < nk) {
                            wait_vmcnt<0>();
                            __builtin_amdgcn_s_barrier();
#pragma unroll
                            for (int r = 0; r < NR; ++r) read_one(r, nstage, 0, nxt);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        stage = nstage;
        lstage = lstage + 1 == S ? 0 : lstage + 1;
    };
    int it = 0;
    for (; it + AHEAD < nk; ++it) block(it, std::true_type{});
    for (; it < nk; ++it) block(it, std::false_type{});

    // acc[i][j][v]: row m = (v/4)*8 + (lane/32)*4 + v%4, column n = lane%32 of the 32x32 tile.
    const int mrow = m0 + wm + (lane >> 5) * 4;     // + i * 32 + (v / 4) * 8 + v % 4
    const int ncol = n0 + wn + lr;                  // + j * 32
    if (EPI == 1 && !SPLIT) {
        // columns come in blocks of 16: 8 gate, then their 8 up (8 lanes further on).  Of two
        // consecutive rows the gate lane finishes the first and the up lane the second.
        const bool up = lr & 8;
        const int ng = up ? ncol - 8 : ncol;
        TO* dst = out + (size_t)(mrow + (up ? 1 : 0)) * (N / 2) + (size_t)(ng >> 4) * 8 + (ng & 7);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; v += 2) {
                    float first = acc[i][j][v], second = acc[i][j][v + 1];
                    asm volatile("" : "+v"(first), "+v"(second));   // two values, not one indexed by `up`
                    const float got = lane_swap<0x128>(up ? first : second);   // lane ^ 8
                    const float r = swiglu_f(up ? got : first, up ? second : got);
                    const int dm = i * 32 + (v >> 2) * 8 + (v & 3);
                    if (mrow + (up ? 1 : 0) + dm < M && ng + j * 32 < N)
                        store_out<TO>(dst + (size_t)dm * (N / 2) + j * 16, r);
                }
    } else {
        using TS = typename std::conditional<SPLIT, float, TO>::type;
        const bool tilewise = SPLIT && compact;    // addresses inside the tile's own [BM][BN] block
        TS* base = !SPLIT ? (TS*)out
                 : tilewise ? (TS*)(part + ((size_t)blockIdx.y * tile_count + local_tile) * BM * BN)
                            : (TS*)(part + (size_t)blockIdx.y * M * N);
        const size_t ld = tilewise ? BN : N;
        const int r0 = tilewise ? m0 : 0, c0 = tilewise ? n0 : 0;
        if ((ld & 1) == 0) {
            // neighbouring lanes swap every other value, so that a lane holds two adjacent
            // columns of one row and stores them together: even lanes the even v, odd lanes the odd
            const bool odd = lane & 1;
            TS* dst = base + (size_t)(mrow - r0 + (odd ? 1 : 0)) * ld + ((ncol & ~1) - c0);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int v = 0; v < 16; v += 2) {
                        float first = acc[i][j][v], second = acc[i][j][v + 1];
                        asm volatile("" : "+v"(first), "+v"(second));   // two values, not one indexed by `odd`
                        const float got = lane_swap<0xB1>(odd ? first : second);   // lane ^ 1
                        const int dm = i * 32 + (v >> 2) * 8 + (v & 3);
                        if (mrow + (odd ? 1 : 0) + dm < M && (ncol & ~1) + j * 32 < N)
                            store_pair<TS>(dst + (size_t)dm * ld + j * 32, odd ? got : first, odd ? second : got);
                    }
        } else {
            TS* dst = base + (size_t)(mrow - r0) * ld + (ncol - c0);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int dm = i * 32 + (v >> 2) * 8 + (v & 3);
                        if (mrow + dm < M && ncol + j * 32 < N)
                            store_out<TS>(dst + (size_t)dm * ld + j * 32, acc[i][j][v]);
                    }
        }
    }
}

// out = sum over the shares of part[s][M][N], added in the order of s; EPI as in the products
template <int EPI, typename TO>
__global__ void splitk_reduce_kernel(const float* __restrict__ part, TO* __restrict__ out, int M, int N,
                                     int S) {
    const size_t MN = (size_t)M * N;
    if (EPI == 0) {
        for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < MN;
             idx += (size_t)gridDim.x * blockDim.x) {
            float t = 0.f;
            for (int s = 0; s < S; ++s) t += part[s * MN + idx];
            store_out<TO>(out + idx, t);
        }
    } else {
        const int half = N / 2;
        for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < (size_t)M * half;
             idx += (size_t)gridDim.x * blockDim.x) {
            const size_t m = idx / half;
            const int c = (int)(idx - m * half);
            const size_t gi = m * N + (size_t)(c >> 3) * 16 + (c & 7);
            float g = 0.f, u = 0.f;
            for (int s = 0; s < S; ++s) { g += part[s * MN + gi]; u += part[s * MN + gi + 8]; }
            store_out<TO>(out + idx, swiglu_f(g, u));
        }
    }
}

// out = sum over the shares of the tiles [tile_base, tile_base + count) that were written tile by
// tile, part[s][tile - tile_base][BM][BN], added in the order of s; EPI as in the products.
// One workgroup per tile and 2048 of its elements.
template <int EPI, typename TO>
__global__ __launch_bounds__(256) void tail_reduce_kernel(const float* __restrict__ part, TO* __restrict__ out,
                                                          int M, int N, int BM, int BN, int tiles_m,
                                                          int tile_base, int count, int S) {
    const int local = blockIdx.x, tile = tile_base + local;
    const int m0 = (tile % tiles_m) * BM, n0 = (tile / tiles_m) * BN;
    const size_t area = (size_t)BM * BN;
    const float* src = part + (size_t)local * area;
    for (int e = blockIdx.y * 2048 + threadIdx.x; e < min((int)area, (blockIdx.y + 1) * 2048); e += 256) {
        const int row = e / BN, col = e - row * BN;
        const int m = m0 + row, n = n0 + col;
        if (m >= M || n >= N) continue;
        if (EPI == 0) {
            float t = 0.f;
            for (int s = 0; s < S; ++s) t += src[(size_t)s * count * area + e];
            store_out<TO>(out + (size_t)m * N + n, t);
        } else if ((n & 15) < 8) {                     // a gate column; its up column lies 8 further on
            float g = 0.f, u = 0.f;
            for (int s = 0; s < S; ++s) {
                g += src[(size_t)s * count * area + e];
                u += src[(size_t)s * count * area + e + 8];
            }
            store_out<TO>(out + (size_t)m * (N / 2) + (size_t)(n >> 4) * 8 + (n & 7), swiglu_f(g, u));
        }
    }
}

// The tile shapes of the tiled kernel.  TILE_AUTO picks by size; the others are forced through
// lc_gemm_bf16_force_tile (tests and tuning).
enum : int { TILE_AUTO = -1, TILE_64x128 = 0, TILE_128x128 = 1, TILE_256x128 = 2, TILE_256x192 = 3, TILE_256x256 = 4,
              TILE_192x128 = 5, TILE_192x256 = 6, TILE_64x64 = 7, TILE_64x96 = 8, TILE_192x320 = 9, TILE_64x224 = 10,
              TILE_64x128_ONE = 11, TILE_64x160 = 12, TILE_COUNT = 13 };
static thread_local int g_force_tile = TILE_AUTO;   // the switches are per thread: a test that flips one
                                                    // never changes what an engine's thread launches
#define kCUs (::lc::device_cus())   // the GPU's compute units: they steer the tile plans only

static int tile_bm(int t) {
    return (t == TILE_64x128 || t == TILE_64x64 || t == TILE_64x96 || t == TILE_64x224 || t == TILE_64x128_ONE || t == TILE_64x160) ? 64 : t == TILE_128x128 ? 128 : (t == TILE_192x128 || t == TILE_192x256 || t == TILE_192x320) ? 192 : 256;
}
static int tile_bn(int t) {
    return (t == TILE_256x256 || t == TILE_192x256) ? 256 : t == TILE_192x320 ? 320 : t == TILE_256x192 ? 192 : t == TILE_64x64 ? 64 : t == TILE_64x96 ? 96 : t == TILE_64x224 ? 224 : t == TILE_64x160 ? 160 : 128;
}
static long long tile_count(int t, int M, int N) {
    return (long long)((M + tile_bm(t) - 1) / tile_bm(t)) * ((N + tile_bn(t) - 1) / tile_bn(t));
}

// The shapes with 192 or 256 rows run one workgroup to a CU, so their tiles go through the CUs in
// rounds of kCUs.  When the last round would be less than half full, its tiles are cut along K
// into `shares` parts each (written tile by tile, summed by tail_reduce_kernel), which fills
// that round's CUs with shorter pieces: rest tiles, shares parts (0, 1: no such tail).
struct TailPlan {
    int rest, shares;
};
static TailPlan tail_plan(int t, int M, int N, int K) {
    TailPlan none = {0, 1};
    if (tile_bm(t) < 192) return none;
    const long long tiles = tile_count(t, M, N);
    const int rest = (int)(tiles % kCUs), nk = K / TL_K;
    if (tiles < kCUs || rest == 0 || rest > kCUs / 2 || nk < 16) return none;
    int shares = kCUs / rest;
    if (shares > nk / 8) shares = nk / 8;
    if (shares < 2) return none;
    TailPlan plan = {rest, shares};
    return plan;
}

// Into how many shares of K a product with this tile is cut as a whole (1: not at all): as many
// as it takes to give every CU about two workgroups when whole-K tiles would be too few.  Only
// the small tiles are cut as a whole; the shares are summed by splitk_reduce_kernel, or by
// whoever takes the partial sums (lc_gemm_bf16_partials).  The tile of 64 x 64 is for up to 64
// rows: cut, it makes half as many shares as the tile of 64 x 128 for the same number of
// workgroups (64 x 4096 x 4096 and the norm that sums its shares: 17.8 instead of 23.5 us;
// 64 x 6144 x 4096 and the sum of its shares: 16.4 instead of 19.6); whole, it saves the kernel
// that sums (see pick_tile).
static thread_local int g_small_partials = 1;   // 0: shares that are handed on come from 64 x 128 tiles (tests, tuning)
static bool whole_k_64x64(int M, int N, int K) {
    const long long tiles64 = tile_count(TILE_64x64, M, N);
    return (tiles64 >= kCUs && tiles64 <= 3 * kCUs) || (K <= 2048 && tiles64 >= 48);
}
// by how many k-blocks a workgroup's start moves per tile where the tiles form a single row (see the
// kernel); measured at 64 x 24576 x 4096 in tiles of 64 x 96: 0: 46.9 us, 1: 41.2, 3: 58.8, 5 to 31
// (odd): 37.0 to 38.2
static thread_local int g_skew = 17;
static thread_local int g_force_shares = 0;   // > 0: the small tiles are cut along K this many ways (tests, tuning)
static int shares_for(int t, int M, int N, int K, bool partials_wanted = false) {
    if (t != TILE_64x128 && t != TILE_128x128 && t != TILE_64x64) return 1;
    if (g_force_shares > 0) return g_force_shares <= K / TL_K ? g_force_shares : K / TL_K;
    if (t == TILE_64x64 && g_force_tile == TILE_AUTO && !partials_wanted && whole_k_64x64(M, N, K)) return 1;
    const long long tiles = tile_count(t, M, N);
    if (tiles >= 400) return 1;
    const int nk = K / TL_K;
    int S = (int)((480 + tiles / 2) / tiles);
    if (S > nk / 4) S = nk / 4;
    return S < 1 ? 1 : S;
}

// The tile for a product with M > 16.  Up to 64 rows: a 64-row tile.  Beyond: the shape with
// the least estimated time in microseconds.  A CU works through a round of tiles in
// (tile area) x K x 2 / (4.63 MFLOP/us x the shape's relative rate) (measured at K = 4096: larger
// tiles move fewer bytes per product) and 3 us to start and end.  A last round of a one-a-CU shape
// that is cut along K takes its share of that, plus the time to write and read its float32
// partial tiles (about 4 TB/s) and to start two more kernels.  A small tile cut along K as a
// whole pays for its partial sums likewise, unless the caller takes them as they are
// (partials_wanted).
static int pick_tile(int M, int N, int K, bool partials_wanted = false) {
    if (g_force_tile != TILE_AUTO) return g_force_tile;
    if (M <= 64) {
        // Tiles of 64 x 64 and whole K where they fill the CUs once to three times, or where K
        // is so short that a second kernel to sum shares costs more than idle CUs (measured:
        // 64 x 24576 x 4096 with SwiGLU 47 instead of 52 us, 64 x 6144 x 1024 9 instead of 11);
        // tiles of 64 x 64 cut along K where there are few of them, and for shares that are
        // handed on; else tiles of 64 x 128, cut where they are few.
        if (partials_wanted) return g_small_partials ? TILE_64x64 : TILE_64x128;
        // Where tiles of 64 x 64 would go through the CUs in more than one round (every CU's way
        // from L2 carries the tile's rows of x and of w, and the CUs with the most tiles set the
        // time), wider tiles that make a single round carry less per CU: one workgroup of two
        // waves a CU, with a deep ring of stages in place of a second workgroup.  The narrowest
        // of the widths 96, 128, 160 and 224 that fits N into one round is taken (64 x 24576 x
        // 4096 with SwiGLU: 384 tiles of 64 x 64 49.3 us, 256 of 64 x 96 37.5; 64 x 51200 x 5120:
        // 400 tiles of 64 x 128 in two rounds 109 us, 229 of 64 x 224 96).
        const long long tiles64 = tile_count(TILE_64x64, M, N);
        if (tiles64 > kCUs && K >= 1024) {
            for (const int t : {TILE_64x96, TILE_64x128_ONE, TILE_64x160, TILE_64x224})
                if (tile_count(t, M, N) <= kCUs) return t;
        }
        if (whole_k_64x64(M, N, K) || tiles64 <= 128) return TILE_64x64;
        return TILE_64x128;
    }
    // (tiles of 64 x 128 for 65 to 128 rows: every tile of w's rows reads all of x again, 96 x
    // 24576 x 4096 with SwiGLU takes 57 us in them and 52 as 192 tiles of 192 x 128 in one round,
    // 128 rows 62 and 50)
    const double rate[TILE_COUNT] = {0.55, 0.82, 0.90, 0.94, 1.0, 0.87, 0.94, 0.5, 0.5, 0.97, 0.6, 0.6, 0.6};
    int best = -1;
    double best_cost = 0.0;
    const int candidates[] = {TILE_64x128, TILE_128x128, TILE_256x128, TILE_256x192, TILE_256x256, TILE_192x128,
                              TILE_192x256, TILE_192x320, TILE_64x64};
    for (const int t : candidates) {
        if (t == TILE_64x128 && M > 128) continue;
        // 64 x 64 above 256 rows: for the narrow products of a portion of a prompt, which have few
        // larger tiles (2,048 x 1024 x 2048 with the norm that follows: 24.6 us in 512 whole tiles of
        // 64 x 64, 31.2 as tiles of 128 x 128 cut along K four ways; 576 x 1024 x 3072 18.7 against 22.3)
        // (up to 256 rows only for a w of up to 32 MB: 128 x 4096 x 4096 with its norm 19.2 us against 21.1 in
        // tiles of 64 x 128; on a large w every tile of 64 rows of w reads all of x again: 128 x 24576 x 4096
        // 61.8 against 50.8 in tiles of 192 x 128.  Measured over the four products of six model sizes at 96 to
        // 4,096 rows, the shape picked is within 8 % of the best of all shapes in 208 of 216 cases.)
        if (t == TILE_64x64 && M <= 256 && (long long)N * K > (1ll << 24)) continue;
        const long long tiles = tile_count(t, M, N);
        const double area = (double)tile_bm(t) * tile_bn(t);
        // (tiles of 64 x 64 do better than their rate on a small w, which stays in the caches)
        const double r = (t == TILE_64x64 && (long long)N * K <= (1ll << 24)) ? 0.62 : rate[t];
        const double work_us = area * K * 2.0 / (4.63e6 * r);
        double cost;
        if (tile_bm(t) >= 192) {
            const double round_us = work_us + 3.0;
            const TailPlan tail = tail_plan(t, M, N, K);
            if (tail.shares > 1)
                cost = (double)(tiles / kCUs) * round_us + round_us / tail.shares +
                       (double)tail.rest * tail.shares * area * 8.0 / 4.0e6 + 10.0;
            else
                cost = (double)((tiles + kCUs - 1) / kCUs) * round_us;
        } else {
            const int S = shares_for(t, M, N, K);
            cost = (double)((tiles * S + kCUs - 1) / kCUs) * (work_us / S + 3.0);
            if (S > 1) cost += (double)M * N * S * (partials_wanted ? 4.0 : 8.0) / 4.0e6 + (partials_wanted ? 0.0 : 10.0);
        }
        cost += 1e-6 * tiles * area * K / 4.63e6;      // equal otherwise: the shape that covers less beyond M x N
        if (best < 0 || cost < best_cost) { best = t; best_cost = cost; }
    }
    return best;
}

static int splitk_shares(int M, int N, int K, bool partials_wanted = false) {
    if (M <= 16) return 1;
    return shares_for(pick_tile(M, N, K, partials_wanted), M, N, K, partials_wanted);
}

// float32 words of workspace that the product needs (0: none)
static long long workspace_words(int M, int N, int K) {
    if (M <= 16 && g_force_tile == TILE_AUTO) return 0;
    const int t = pick_tile(M, N, K);
    const int S = splitk_shares(M, N, K);
    if (S > 1) return (long long)S * M * N;
    const TailPlan tail = tail_plan(t, M, N, K);
    if (tail.shares > 1) return (long long)tail.shares * tail.rest * tile_bm(t) * tile_bn(t);
    return 0;
}

template <int MT, int NT, int WAVES, int UNROLL, int EPI, bool SCALE, int XR, typename TO>
static void launch_skinny(const bf16* x, const bf16* w, TO* out, int M, int N, int K, int rows,
                          SkinnyFuse fuse, int workgroups, hipStream_t s) {
    gemm_skinny_kernel<MT, NT, WAVES, UNROLL, EPI, SCALE, XR, TO><<<workgroups, WAVES * 64, 0, s>>>(
        x, w, out, M, N, K, rows, fuse);
}

// The skinny kernel's shape for M <= 16 rows.  Measured: with one or two rows of x a deeper
// unroll keeps more of w in flight.  From a few rows on, fetching x costs a good part of what w
// costs: where there are more tiles than CUs and K allows it, one workgroup a CU takes several
// tiles and keeps x in registers (its registers leave room for one workgroup a CU only, which
// costs more than x does below 7 rows, unless the tiles are so few that the plain shape would
// not fill the CUs twice); else, from about 12 rows on, two row tiles per workgroup share x
// (only where that still leaves every CU two workgroups).
enum : int { SKINNY_DEEP = 0, SKINNY_PLAIN = 1, SKINNY_WIDE = 2, SKINNY_KEEP_X = 3 };
constexpr int SK_KEEP_MAX = 3;   // k blocks of x per wave that fit in registers beside w's
static thread_local int g_force_skinny = -1;
static int skinny_shape(int M, int N, int K) {
    if (g_force_skinny >= 0 && (g_force_skinny != SKINNY_KEEP_X || K <= SK_KEEP_MAX * 16 * SK_KBLOCK))
        return g_force_skinny;
    if (M <= 2) return SKINNY_DEEP;
    const int tiles = (N + 15) / 16;
    if (K <= SK_KEEP_MAX * 16 * SK_KBLOCK && tiles > kCUs && (M >= 7 || tiles <= 2 * kCUs)) return SKINNY_KEEP_X;
    if (M >= 12 && N >= 32 * 2 * kCUs) return SKINNY_WIDE;
    return SKINNY_PLAIN;
}
// How a product of up to 16 rows is laid over the GPU: the kernel's shape, the rows of w of a
// work item, the number of items (also the number of pieces that epilogue 2 writes) and the
// number of workgroups.  A workgroup streams its rows of w at the pace of memory, so what
// counts is that every CU gets the same number of rows.  Items of 16 (or 32) rows do that when
// their number is a multiple of the CUs or many times it; at 320 items for 256 CUs a quarter of
// the CUs would work twice as long as the rest.  Then N is cut into items of fewer rows, as
// many as give every CU the same number (the SwiGLU epilogue needs whole blocks of 16 rows and
// keeps them).
struct SkinnyPlan {
    int shape, rows, items, groups;
    bool runs;      // the kernel that reads w in runs of 1 KB
};
static thread_local int g_even_rows = 1;
static thread_local int g_runs = 1;

// Whether gemm_runs_kernel keeps its x in registers for all of a workgroup's tiles (XS = 8) or
// fetches it stage by stage into a ring of registers (XS = 0).
static bool runs_keeps_x(const SkinnyPlan& p, int K) { return K / SR_K <= 8 && p.items > p.groups; }

// The XS = 0 form loads x by inline assembly into registers that it reads only after a counted
// wait; in between, the compiler takes those registers to hold values already.  That is sound
// as long as the ring stays in registers: were one of them spilled to scratch memory, the spill
// would store whatever the register held before the load landed.  So the compiled kernels are
// asked, once: if any XS = 0 instantiation uses scratch memory (or cannot be asked), that form
// is not run and the plain skinny kernel takes its sizes.
static int runs_ring_state() {       // 1: in registers, 0: spilled, -1: could not ask
    static const int state = [] {
        const void* kernels[] = {
            (const void*)gemm_runs_kernel<0, false, 0, bf16>, (const void*)gemm_runs_kernel<0, false, 0, float>,
            (const void*)gemm_runs_kernel<1, false, 0, bf16>, (const void*)gemm_runs_kernel<1, false, 0, float>,
            (const void*)gemm_runs_kernel<2, false, 0, float>,
            (const void*)gemm_runs_kernel<0, true, 0, bf16>, (const void*)gemm_runs_kernel<1, true, 0, bf16>,
        };
        for (const void* kernel : kernels) {
            hipFuncAttributes attr;
            if (hipFuncGetAttributes(&attr, kernel) != hipSuccess) {
                (void)hipGetLastError();
                return -1;
            }
            if (attr.localSizeBytes != 0) return 0;
        }
        return 1;
    }();
    return state;
}
static bool runs_ring_in_registers() { return runs_ring_state() == 1; }

static SkinnyPlan skinny_plan(int M, int N, int K, int epilogue) {
    SkinnyPlan p;
    p.runs = false;
    // (measured at 8 rows: 201 MB of w 41.8 -> 38.7 us, 100 MB 24.8 -> 22.3, 1.2 GB 221 -> 213; 50 MB 12.4 -> 13.5 and
    // 34 MB 9.8 -> 10.1: the ring's start and the barrier of every stage cost the small ones more than the runs gain)
    // With one or two rows of x the kernel above, one tile a workgroup, is the faster one (1.2 GB of w: 196 against 206 us).
    // (a long K, as the down products have, gains from a smaller w on: 2560 x 9728 16.0 instead of 17.7 us at 8 rows,
    // 2048 x 6144 12.0 instead of 13.1)
    const bool large = (long long)N * K >= (1ll << 25) || (K >= 6144 && (long long)N * K >= (1ll << 23));
    if (g_runs && g_force_skinny < 0 && K % SR_K == 0 && (g_runs > 1 || (M >= 4 && large))) {
        // tiles of 16 rows, or of as many as give every CU the same number (the SwiGLU epilogue keeps whole blocks of 16)
        p.runs = true;
        p.shape = SKINNY_PLAIN;
        p.rows = 16;
        p.items = (N + 15) / 16;
        const int per_cu = (p.items + kCUs - 1) / kCUs;
        if (g_even_rows && epilogue != 1 && p.items > kCUs && p.items % kCUs != 0 && per_cu <= 4) {
            p.rows = (N + kCUs * per_cu - 1) / (kCUs * per_cu);
            p.items = (N + p.rows - 1) / p.rows;
        }
        p.groups = p.items < kCUs ? p.items : kCUs;
        // the form of the kernel that keeps x in a ring of registers filled by hand-counted loads
        // runs only when the compiler has put that ring into registers (see runs_ring_in_registers)
        if (runs_keeps_x(p, K) || runs_ring_in_registers()) return p;
        p.runs = false;
    }
    p.shape = skinny_shape(M, N, K);
    p.rows = p.shape == SKINNY_WIDE ? 32 : 16;
    p.items = (N + p.rows - 1) / p.rows;
    const bool keep = p.shape == SKINNY_KEEP_X;
    if (g_even_rows && g_force_skinny < 0 && epilogue != 1 && p.items > kCUs && p.items % kCUs != 0) {
        const int per_cu = (p.items + kCUs - 1) / kCUs;            // items of the busiest CU as it is
        if (keep && per_cu <= 4) {
            p.rows = (N + kCUs * per_cu - 1) / (kCUs * per_cu);    // x stays in registers: small items cost nothing
        } else if (!keep && p.shape != SKINNY_WIDE && per_cu == 2 && M > 2) {
            p.shape = SKINNY_WIDE;                                 // one item a CU, of up to 32 rows: x is fetched once a CU
            p.rows = (N + kCUs - 1) / kCUs;
        } else if (!keep && p.shape != SKINNY_WIDE && per_cu <= 4) {
            p.rows = (N + kCUs * per_cu - 1) / (kCUs * per_cu);
        }
        p.items = (N + p.rows - 1) / p.rows;
    }
    p.groups = keep ? (p.items < kCUs ? p.items : kCUs) : p.items;   // keep-x: one workgroup a CU fits
    return p;
}
static int skinny_tiles(int M, int N, int K, int epilogue) { return skinny_plan(M, N, K, epilogue).items; }

template <int EPI, bool SCALE, typename TO>
static void launch_skinny_any(const bf16* x, const bf16* w, TO* out, int M, int N, int K, SkinnyFuse fuse,
                              hipStream_t s) {
    const SkinnyPlan p = skinny_plan(M, N, K, EPI);
    if (p.runs) {
        // x stays in registers where a workgroup has several tiles to use it for
        if (runs_keeps_x(p, K)) gemm_runs_kernel<EPI, SCALE, 8, TO><<<p.groups, 1024, 0, s>>>(x, w, out, M, N, K, p.rows, fuse);
        else gemm_runs_kernel<EPI, SCALE, 0, TO><<<p.groups, 1024, 0, s>>>(x, w, out, M, N, K, p.rows, fuse);
        return;
    }
    const int per_wave = (K / SK_KBLOCK + 15) / 16;
    switch (p.shape) {
    case SKINNY_DEEP: launch_skinny<1, 1, 16, 4, EPI, SCALE, 0, TO>(x, w, out, M, N, K, p.rows, fuse, p.groups, s); break;
    case SKINNY_WIDE: launch_skinny<1, 2, 16, 2, EPI, SCALE, 0, TO>(x, w, out, M, N, K, p.rows, fuse, p.groups, s); break;
    case SKINNY_KEEP_X:
        if (per_wave == 1) launch_skinny<1, 1, 16, 1, EPI, SCALE, 1, TO>(x, w, out, M, N, K, p.rows, fuse, p.groups, s);
        else if (per_wave == 2) launch_skinny<1, 1, 16, 1, EPI, SCALE, 2, TO>(x, w, out, M, N, K, p.rows, fuse, p.groups, s);
        else launch_skinny<1, 1, 16, 1, EPI, SCALE, 3, TO>(x, w, out, M, N, K, p.rows, fuse, p.groups, s);
        break;
    default:          launch_skinny<1, 1, 16, 2, EPI, SCALE, 0, TO>(x, w, out, M, N, K, p.rows, fuse, p.groups, s); break;
    }
}

template <int BM, int BN, int STAGES, int EPI, typename TO, int WM = 2, int WN = 2>
static int launch_tiled(const bf16* x, const bf16* w, TO* out, float* workspace, int M, int N, int K,
                        int shares, TailPlan tail, hipStream_t s) {
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const int tiles = tiles_m * tiles_n;
    if (shares == 1 && tail.shares <= 1) {
        gemm_tiled_kernel<BM, BN, STAGES, EPI, false, TO, WM, WN><<<tiles, 64 * WM * WN, 0, s>>>(
            x, w, out, nullptr, M, N, K, tiles_m, 0, tiles, 0, g_skew);
        LC_LAUNCH_CHECK("gemm_tiled");
        return 0;
    }
    if constexpr (WM != 2 || WN != 2) {
        LC_CHECK(false, "gemm_bf16: the tile %dx%d is not cut along K", BM, BN);
        return 0;
    } else {
    LC_CHECK(workspace, "gemm_bf16: M=%d N=%d K=%d needs a workspace", M, N, K);
    if constexpr (BM >= 192) {
        LC_CHECK(shares == 1 && tail.rest > 0 && tail.rest < tiles, "gemm_bf16: bad tail for tile %dx%d", BM, BN);
        const int whole = tiles - tail.rest;
        gemm_tiled_kernel<BM, BN, STAGES, EPI, false, TO><<<whole, 256, 0, s>>>(
            x, w, out, nullptr, M, N, K, tiles_m, 0, whole, 0, g_skew);
        LC_LAUNCH_CHECK("gemm_tiled");
        gemm_tiled_kernel<BM, BN, STAGES, 0, true, TO><<<dim3(tail.rest, tail.shares), 256, 0, s>>>(
            x, w, out, workspace, M, N, K, tiles_m, whole, tail.rest, 1, g_skew);
        LC_LAUNCH_CHECK("gemm_tiled");
        tail_reduce_kernel<EPI, TO><<<dim3(tail.rest, (BM * BN + 2047) / 2048), 256, 0, s>>>(
            workspace, out, M, N, BM, BN, tiles_m, whole, tail.rest, tail.shares);
        LC_LAUNCH_CHECK("tail_reduce");
        return 0;
    } else {
        LC_CHECK(tail.shares <= 1, "gemm_bf16: tile %dx%d has no tail", BM, BN);
        gemm_tiled_kernel<BM, BN, STAGES, 0, true, TO><<<dim3(tiles, shares), 256, 0, s>>>(
            x, w, out, workspace, M, N, K, tiles_m, 0, tiles, 0, g_skew);
        LC_LAUNCH_CHECK("gemm_tiled");
        const size_t work = EPI ? (size_t)M * N / 2 : (size_t)M * N;
        splitk_reduce_kernel<EPI, TO><<<(int)((work + 255) / 256), 256, 0, s>>>(workspace, out, M, N, shares);
        LC_LAUNCH_CHECK("splitk_reduce");
        return 0;
    }
    }
}

template <int EPI, typename TO>
static int launch_bf16(const bf16* x, const bf16* w, TO* out, float* workspace, int M, int N, int K,
                       hipStream_t s) {
    if (M <= 16 && g_force_tile == TILE_AUTO) {
        launch_skinny_any<EPI, false, TO>(x, w, out, M, N, K, SkinnyFuse{}, s);
        LC_LAUNCH_CHECK("gemm_skinny");
        return 0;
    }
    const int shares = splitk_shares(M, N, K);
    const int tile = pick_tile(M, N, K);
    const TailPlan tail = tail_plan(tile, M, N, K);
    switch (tile) {
    case TILE_64x128:  return launch_tiled<64, 128, 3, EPI, TO>(x, w, out, workspace, M, N, K, shares, tail, s);
    case TILE_128x128: return launch_tiled<128, 128, 2, EPI, TO>(x, w, out, workspace, M, N, K, shares, tail, s);
    case TILE_256x128: return launch_tiled<256, 128, 3, EPI, TO>(x, w, out, workspace, M, N, K, shares, tail, s);
    case TILE_256x192: return launch_tiled<256, 192, 2, EPI, TO>(x, w, out, workspace, M, N, K, shares, tail, s);
    case TILE_192x128: return launch_tiled<192, 128, 3, EPI, TO>(x, w, out, workspace, M, N, K, shares, tail, s);
    case TILE_192x256: return launch_tiled<192, 256, 2, EPI, TO>(x, w, out, workspace, M, N, K, shares, tail, s);
    case TILE_64x64:   return launch_tiled<64, 64, 3, EPI, TO>(x, w, out, workspace, M, N, K, shares, tail, s);
    case TILE_64x96:   return launch_tiled<64, 96, 6, EPI, TO, 2, 1>(x, w, out, workspace, M, N, K, shares, tail, s);
    case TILE_192x320: return launch_tiled<192, 320, 2, EPI, TO>(x, w, out, workspace, M, N, K, shares, tail, s);
    case TILE_64x224:  return launch_tiled<64, 224, 4, EPI, TO, 2, 1>(x, w, out, workspace, M, N, K, shares, tail, s);
    case TILE_64x128_ONE: return launch_tiled<64, 128, 5, EPI, TO, 2, 1>(x, w, out, workspace, M, N, K, shares, tail, s);
    case TILE_64x160:  return launch_tiled<64, 160, 4, EPI, TO, 2, 1>(x, w, out, workspace, M, N, K, shares, tail, s);
    default:           return launch_tiled<256, 256, 2, EPI, TO>(x, w, out, workspace, M, N, K, shares, tail, s);
    }
}

}  // namespace lc

using namespace lc;

// Sizes the matrix-core kernels take; everything else goes to the generic kernel.
LC_API int lc_gemm_bf16_supported(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    if (K % SK_KBLOCK != 0) return 0;
    if ((size_t)((M + 63) / 64) * ((N + 127) / 128) > 0x7fffffffu) return 0;
    return 1;
}

// What K must be a multiple of for the matrix-core kernels.
LC_API int lc_gemm_bf16_kblock() { return SK_KBLOCK; }

// Forces the shape of the skinny kernel for every later product of up to 16 rows (0: deep
// unroll, 1: plain, 2: two row tiles of w a workgroup, 3: several tiles a workgroup with x kept
// in registers, where K allows it; -1: choose by size again).  For tests and tuning.
LC_API int lc_gemm_bf16_force_skinny(int shape) {
    LC_CHECK(shape >= -1 && shape <= SKINNY_KEEP_X, "gemm_bf16: no skinny shape %d", shape);
    g_force_skinny = shape;
    return 0;
}

// Forces the tile shape of the tiled kernel for every later product of any M that the calling
// thread launches (-1: choose by size again).  For tests and tuning.
LC_API int lc_gemm_bf16_force_tile(int tile) {
    LC_CHECK(tile >= TILE_AUTO && tile < TILE_COUNT, "gemm_bf16: no tile shape %d", tile);
    g_force_tile = tile;
    return 0;
}

// The tile shape that a product of these sizes goes through (the numbers of lc_gemm_bf16_force_tile;
// -1: up to 16 rows, which the skinny kernels take), and into how many shares of K it is cut;
// partials: as lc_gemm_bf16_partials would do it.  For tests and tuning.
LC_API int lc_gemm_bf16_tile(int M, int N, int K, int partials) {
    if (!lc_gemm_bf16_supported(M, N, K) || (M <= 16 && g_force_tile == TILE_AUTO)) return -1;
    return pick_tile(M, N, K, partials != 0);
}

// float32 words of workspace that lc_gemm_bf16 needs for these sizes (0: none).
LC_API long long lc_gemm_bf16_workspace(int M, int N, int K) {
    if (!lc_gemm_bf16_supported(M, N, K)) return 0;
    return workspace_words(M, N, K);
}

// epilogue 0: out[M, N] = x . w^T.  epilogue 1 (SwiGLU): the rows of w come in blocks of 16,
// 8 gate rows followed by their 8 up rows; out[M, N / 2] = silu(gate) * up.
// workspace: lc_gemm_bf16_workspace(M, N, K) float32 words (may be null when that is 0).
LC_API int lc_gemm_bf16(const void* x, const void* w, void* out, int out_dt, int M, int N, int K,
                        int epilogue, float* workspace, hipStream_t stream) {
    LC_CHECK(lc_gemm_bf16_supported(M, N, K), "gemm_bf16: sizes M=%d N=%d K=%d are not supported "
             "(K must be a multiple of %d)", M, N, K, SK_KBLOCK);
    LC_CHECK(x && w && out, "gemm_bf16: null pointer");
    LC_CHECK(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_bf16: operands must be 16-byte aligned");
    LC_CHECK((uintptr_t)out % 8 == 0 && (uintptr_t)workspace % 8 == 0, "gemm_bf16: out and workspace must be 8-byte aligned");
    LC_CHECK(epilogue == 0 || (epilogue == 1 && N % 16 == 0),
             "gemm_bf16: the SwiGLU epilogue needs N (%d) to be a multiple of 16", N);
    const bf16* xb = (const bf16*)x;
    const bf16* wb = (const bf16*)w;
    if (out_dt == DT_BF16)
        return epilogue ? launch_bf16<1, bf16>(xb, wb, (bf16*)out, workspace, M, N, K, stream)
                        : launch_bf16<0, bf16>(xb, wb, (bf16*)out, workspace, M, N, K, stream);
    if (out_dt == DT_F32)
        return epilogue ? launch_bf16<1, float>(xb, wb, (float*)out, workspace, M, N, K, stream)
                        : launch_bf16<0, float>(xb, wb, (float*)out, workspace, M, N, K, stream);
    LC_CHECK(false, "gemm_bf16: unknown output dtype %d", out_dt);
    return 0;
}

// ------------------------------------------------------------------- norms folded into products
// For steps of up to 16 rows (decode), where a norm kernel costs its start and nothing else.
// The residual stream h [M, H] is float32.  A "prepared norm" of h for a norm weight g is the
// pair (xg = bf16(h * g) [M, H], pieces [count][stride] of every row's sum of squares): what is
// missing is each row's factor rsqrt(mean(h^2) + eps), which a product can apply to its sums.
// The pieces of row m lie at [piece][m] with lc_gemm_bf16_piece_stride(M) floats per piece.

// 0: work items of 16 or 32 rows whatever N is; 1 (the default): N cut into equal items where
// that gives every CU the same number of rows.  For tests and tuning.
// Whether products of up to 16 rows read w in runs of 1 KB through LDS: where K allows it and w
// is large enough to gain (1, the default), wherever K allows it (2), never (0).  For tests
// and tuning.
LC_API int lc_gemm_bf16_runs(int on) {
    g_runs = on;
    return 0;
}

// 1: the form of the runs kernel that keeps x in a ring of registers filled by hand-counted loads
// is compiled without scratch memory and may run; 0: it spills and is not run; -1: the kernels
// could not be asked (no device) and it is not run.
LC_API int lc_gemm_bf16_runs_ring_ok() { return runs_ring_state(); }

LC_API int lc_gemm_bf16_even_rows(int on) {
    g_even_rows = on ? 1 : 0;
    return 0;
}

// The step of the k-block skew of products with a single row of tiles (0: none; 17 by default).
// For tests and tuning.
LC_API int lc_gemm_bf16_skew(int step) {
    LC_CHECK(step >= 0, "gemm_bf16: bad skew %d", step);
    g_skew = step;
    return 0;
}

// > 0: products that go through the small tiles (64 x 64, 64 x 128, 128 x 128) are cut along K
// this many ways, whatever their size; 0: by size again.  For tests and tuning.
LC_API int lc_gemm_bf16_force_shares(int shares) {
    LC_CHECK(shares >= 0 && shares <= 64, "gemm_bf16: %d shares (0 to 64)", shares);
    g_force_shares = shares;
    return 0;
}

// 0: shares that are handed on come from tiles of 64 x 128 also for up to 64 rows.  For tests and tuning.
LC_API int lc_gemm_bf16_small_partials(int on) { g_small_partials = on; return 0; }

LC_API int lc_gemm_bf16_piece_stride(int M) {
    int stride = 1;
    while (stride < M) stride *= 2;
    return stride;
}

// Number of pieces that lc_gemm_bf16_residual writes for these sizes; 0: the fused kernels do
// not take these sizes (more than 16 rows, K not a multiple of 128, a forced tile shape, more
// pieces than a scaled product reads).
LC_API int lc_gemm_bf16_residual_pieces(int M, int N, int K) {
    if (!lc_gemm_bf16_supported(M, N, K) || M > 16 || g_force_tile != TILE_AUTO) return 0;
    const int pieces = skinny_tiles(M, N, K, 2);
    return pieces <= SK_MAX_PIECES ? pieces : 0;
}

// resid [M, N] += x [M, K] . w [N, K]^T (float32, in place); next_x [M, N] = bf16(resid * next_w);
// next_pieces [lc_gemm_bf16_residual_pieces(M, N, K)][stride]: sums of squares of the new rows.
LC_API int lc_gemm_bf16_residual(const void* x, const void* w, float* resid, const float* next_w,
                                 void* next_x, float* next_pieces, int M, int N, int K,
                                 hipStream_t stream) {
    LC_CHECK(lc_gemm_bf16_residual_pieces(M, N, K) > 0,
             "gemm_bf16_residual: sizes M=%d N=%d K=%d are not supported", M, N, K);
    LC_CHECK(x && w && resid && next_w && next_x && next_pieces, "gemm_bf16_residual: null pointer");
    LC_CHECK(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_bf16_residual: operands must be 16-byte aligned");
    SkinnyFuse fuse{};
    fuse.resid = resid;
    fuse.next_w = next_w;
    fuse.next_x = (bf16*)next_x;
    fuse.next_partials = next_pieces;
    fuse.stride = lc_gemm_bf16_piece_stride(M);
    launch_skinny_any<2, false, float>((const bf16*)x, (const bf16*)w, (float*)nullptr, M, N, K, fuse, stream);
    LC_LAUNCH_CHECK("gemm_skinny");
    return 0;
}

// Whether lc_gemm_bf16_scaled_rows takes these sizes.
LC_API int lc_gemm_bf16_scaled_rows_supported(int M, int N, int K) {
    return lc_gemm_bf16_supported(M, N, K) && M <= 16 && g_force_tile == TILE_AUTO;
}

// out = (x . w^T) with row m scaled by rsqrt(sum_p pieces[p][m] / K + eps) before the epilogue
// (0: plain, bfloat16 [M, N]; 1: SwiGLU as in lc_gemm_bf16, bfloat16 [M, N / 2]).
LC_API int lc_gemm_bf16_scaled_rows(const void* x, const void* w, void* out, int M, int N, int K,
                                    int epilogue, const float* pieces, int count, float eps,
                                    hipStream_t stream) {
    LC_CHECK(lc_gemm_bf16_scaled_rows_supported(M, N, K),
             "gemm_bf16_scaled_rows: sizes M=%d N=%d K=%d are not supported", M, N, K);
    LC_CHECK(count >= 1 && count <= SK_MAX_PIECES, "gemm_bf16_scaled_rows: %d pieces (at most %d)", count, SK_MAX_PIECES);
    LC_CHECK(x && w && out && pieces, "gemm_bf16_scaled_rows: null pointer");
    LC_CHECK(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_bf16_scaled_rows: operands must be 16-byte aligned");
    LC_CHECK(epilogue == 0 || (epilogue == 1 && N % 16 == 0),
             "gemm_bf16_scaled_rows: the SwiGLU epilogue needs N (%d) to be a multiple of 16", N);
    SkinnyFuse fuse{};
    fuse.scale_partials = pieces;
    fuse.scale_count = count;
    fuse.scale_eps = eps;
    fuse.stride = lc_gemm_bf16_piece_stride(M);
    if (epilogue) launch_skinny_any<1, true, bf16>((const bf16*)x, (const bf16*)w, (bf16*)out, M, N, K, fuse, stream);
    else launch_skinny_any<0, true, bf16>((const bf16*)x, (const bf16*)w, (bf16*)out, M, N, K, fuse, stream);
    LC_LAUNCH_CHECK("gemm_skinny");
    return 0;
}

// ------------------------------------------------------------------ products left as shares
// Where the product of more than 16 rows is cut along K (few tiles, see splitk_shares), the
// shares' float32 sums can be handed on as they are: the norm kernel that adds the product to
// the residual stream sums them itself, in the order of the shares, and the reduction kernel
// and the rounding of the product to bfloat16 fall away.

// Number of shares that lc_gemm_bf16_partials writes for these sizes (0: this product is not cut).
LC_API int lc_gemm_bf16_shares(int M, int N, int K) {
    if (!lc_gemm_bf16_supported(M, N, K) || M <= 16) return 0;
    const int shares = splitk_shares(M, N, K, true);
    return shares > 1 ? shares : 0;
}

// partials [lc_gemm_bf16_shares(M, N, K)][M][N] float32: x . w^T is their sum.
LC_API int lc_gemm_bf16_partials(const void* x, const void* w, float* partials, int M, int N, int K,
                                 hipStream_t stream) {
    const int shares = lc_gemm_bf16_shares(M, N, K);
    LC_CHECK(shares > 1, "gemm_bf16_partials: the product M=%d N=%d K=%d is not cut along K", M, N, K);
    LC_CHECK(x && w && partials, "gemm_bf16_partials: null pointer");
    LC_CHECK(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0) && (uintptr_t)partials % 8 == 0,
             "gemm_bf16_partials: operands must be 16-byte aligned");
    const bf16* xb = (const bf16*)x;
    const bf16* wb = (const bf16*)w;
    if (pick_tile(M, N, K, true) == TILE_64x64) {
        const int tiles_m = (M + 63) / 64, tiles = tiles_m * ((N + 63) / 64);
        gemm_tiled_kernel<64, 64, 3, 0, true, float><<<dim3(tiles, shares), 256, 0, stream>>>(
            xb, wb, nullptr, partials, M, N, K, tiles_m, 0, tiles, 0, g_skew);
    } else if (pick_tile(M, N, K, true) == TILE_64x128) {
        const int tiles_m = (M + 63) / 64, tiles = tiles_m * ((N + 127) / 128);
        gemm_tiled_kernel<64, 128, 3, 0, true, float><<<dim3(tiles, shares), 256, 0, stream>>>(
            xb, wb, nullptr, partials, M, N, K, tiles_m, 0, tiles, 0, g_skew);
    } else {
        const int tiles_m = (M + 127) / 128, tiles = tiles_m * ((N + 127) / 128);
        gemm_tiled_kernel<128, 128, 2, 0, true, float><<<dim3(tiles, shares), 256, 0, stream>>>(
            xb, wb, nullptr, partials, M, N, K, tiles_m, 0, tiles, 0, g_skew);
    }
    LC_LAUNCH_CHECK("gemm_tiled");
    return 0;
}


// out [M, N] (dt: bfloat16 or float32) = the sum of partials [shares][M][N] in their order: what
// lc_gemm_bf16 itself does with the shares of a product that it cuts along K.
LC_API int lc_gemm_bf16_sum_shares(const float* partials, void* out, int dt, int M, int N, int shares,
                                   hipStream_t stream) {
    LC_CHECK(partials && out && M >= 0 && N > 0 && shares >= 1, "gemm_bf16_sum_shares: bad arguments");
    if (M == 0) return 0;
    const size_t work = (size_t)M * N;
    const int blocks = (int)((work + 255) / 256 < 65535 * 16 ? (work + 255) / 256 : 65535 * 16);
    if (dt == DT_BF16) splitk_reduce_kernel<0, bf16><<<blocks, 256, 0, stream>>>(partials, (bf16*)out, M, N, shares);
    else if (dt == DT_F32) splitk_reduce_kernel<0, float><<<blocks, 256, 0, stream>>>(partials, (float*)out, M, N, shares);
    else LC_CHECK(false, "gemm_bf16_sum_shares: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("splitk_reduce");
    return 0;
}
