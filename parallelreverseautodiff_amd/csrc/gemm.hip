// Dense matrix products on the gfx950 matrix cores for the three contractions of
// MatrixMultiplyOperation (src/RMAD/MatrixMultiplyOperation.cs:50-126):
//     forward   C  = A . B        (transA = 0, transB = 0)
//     backward  dA = dC . B^T     (transA = 0, transB = 1)
//     backward  dB = A^T . dC     (transA = 1, transB = 0)
// in double (v_mfma_f64_16x16x4_f64) and float (v_mfma_f32_16x16x4_f32).  They replace the 8 x 8
// shared-memory kernel of src/RMAD/GpuMatrixMultiplyOperation.cs:39-91 and the host-side
// transposed copies it is fed with (:148, :154, :210-248): a transposed operand is read in its
// stored orientation and only its placement in LDS differs.
//
// Shape of one workgroup: 256 threads = 4 wavefronts (2 x 2).  The output tile is 32*WT x 32*WT:
// each wavefront owns WT x WT MFMA tiles of 16 x 16, so a fragment read from LDS feeds WT MFMAs.
// 128 x 128 (WT = 4) is the steady-state shape; the 64 and 32 tiles exist so that products with few
// 128 x 128 tiles still put work on all 256 compute units.  The reduction dimension is cut into
// slabs of 16 KiB per operand (BK = 16 doubles for the 128 tile, 64 for the 32 tile); slabs are
// double-buffered in LDS and global loads run two slabs ahead of the MFMAs.
//
// LDS placement of an operand slab (MN = its rows/columns of the output tile):
//   stored with the reduction index contiguous ("KC": A of the forward, both operands of dA)
//       S[mn][k], row pitch BK elements + 16 bytes, chosen so that the 16 bytes of two neighbouring k
//       of 16 consecutive mn fall into distinct 16-byte bank groups (an XOR-swizzled unpadded
//       layout was measured too: same speed in double, 6 % slower in float because the compiler
//       can no longer merge neighbouring LDS reads; a pitch of one element (double) / two (float) past the
//       power of two, which takes the two-way conflicts that SQ_LDS_BANK_CONFLICT shows for this placement out of
//       the fragment reads but lets the slab be written in 8-byte halves only, was measured as well: nothing at
//       N <= 2048 in double, -2 % at N >= 2048 in float - the conflicts are not what the small tiles wait for);
//   stored with mn contiguous ("MC": B of the forward, both operands of dB)
//       S[k][mn], row pitch MN + 16 elements for the 128 tile; the smaller tiles keep the pitch at MN and
//       rotate row k instead (Slab::mc_shift), so that two of their workgroups fit on a compute unit.
// An MFMA lane (mn = lane % 16, k = lane / 16) reads one element from either placement without
// bank conflicts, so no transposed copy is ever written.
//
// Around the main loop: tiles that hang over the edge of the output clamp their loads and guard their stores
// (only operands whose rows are not 16-byte aligned take the guarded scalar kernels); products with few tiles
// are split along K and reduced inside the kernel by the last workgroup to arrive at a tile (gemm_split_factor,
// gemm_pairs); the epilogue is a plain store, an elementwise pass staged through LDS (bias, activation, upstream
// activation's backward), a per-tile sum, or the cell arithmetic of an LSTM step; a column sum (bias gradient)
// can ride along on extra workgroups of the grid.
#include "common.h"

#include <cstdlib>
#include <type_traits>
#include <cstring>

namespace prad {

typedef double d4_t __attribute__((ext_vector_type(4)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef double d2_t __attribute__((ext_vector_type(2)));

#ifndef PRAD_GEMM_MIX_WT
#define PRAD_GEMM_MIX_WT 4  // largest tile (edge / 32) whose main loop issues its transfers between its MFMAs
#endif
#ifndef PRAD_GEMM_FOLD_K
#define PRAD_GEMM_FOLD_K 512  // float accumulators are folded into a second set every so many elements of K (0: never)
#endif
constexpr int GEMM_THREADS = 256;
constexpr int NUM_XCD = 8;
constexpr int GROUP_M = 8;
constexpr int NV = 4;  // 16-byte vectors per thread per operand slab of full depth, for every tile shape

template <typename T> struct Mfma;
template <> struct Mfma<double> {
    typedef d4_t Acc;
    typedef d2_t Vec;
    static constexpr int VEC = 2;           // elements per 16-byte load
    static constexpr int SLAB_ELEMS = 2048; // elements of one operand slab: MN x BK, 16 KiB
    static constexpr int KPAD = 2;          // padding of a KC slab row (16 bytes)
    static __device__ __forceinline__ Acc run(double a, double b, Acc c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    // Row of the 16 x 16 result held in accumulator element r by lane group g = lane / 16.
    static __device__ __forceinline__ int row(int r, int g) { return 4 * r + g; }
};
template <> struct Mfma<float> {
    typedef f4_t Acc;
    typedef f4_t Vec;
    static constexpr int VEC = 4;
    static constexpr int SLAB_ELEMS = 4096;
    static constexpr int KPAD = 4;
    static __device__ __forceinline__ Acc run(float a, float b, Acc c) {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int row(int r, int g) { return 4 * g + r; }
};

// Geometry of one operand slab for an output tile edge MN = 32 * WT: MN rows/columns by BK of the
// reduction dimension, always 16 KiB, so BK = 16, 32, 64 doubles (32, 64, 128 floats) for the
// 128, 64, 32 tiles: the small tiles, which run with one wavefront per SIMD and cannot hide a
// global-memory round trip behind another workgroup, make four times fewer of them.
// DIV = 2: slabs of half the depth (8 KiB, two vectors per thread), for products of few K slabs whose workgroups
// should rather be three to a compute unit than two.
template <typename T, int WT, int DIV = 1>
struct Slab {
    static constexpr int MN = 32 * WT;
    static constexpr int BK = Mfma<T>::SLAB_ELEMS / MN / DIV;
    static constexpr int NVEC = NV / DIV;                    // 16-byte vectors per thread per slab
    static constexpr int LDK = BK + Mfma<T>::KPAD;  // pitch of a KC row: 16 bytes past a multiple of 128/256/512 bytes
    // MC rows (one k each, MN elements): the 128 tile pads the pitch by 16 elements; the smaller tiles, whose
    // padded slabs would let only one workgroup live on a compute unit, keep the pitch at MN and rotate row k
    // by mc_shift(k) elements instead, which gives the MFMA lane read (16 columns x 4 consecutive k) the same
    // conflict-free bank pattern.
    static constexpr bool ROTATE_MC = WT < 4;
    static constexpr int LDM = ROTATE_MC ? MN : MN + 16;
    static __device__ __forceinline__ int mc_shift(int k) {
        if (!ROTATE_MC) return 0;
        if (sizeof(T) == 8) return 16 * (k & 1);           // a row spans all banks (MN = 32) or twice (64)
        return MN == 32 ? 16 * ((k >> 1) & 1) : 16 * (k & 3);  // floats: rows start 32 banks apart, or at the same bank
    }
    static constexpr int TPR_KC = BK / Mfma<T>::VEC;        // threads covering one KC row
    static constexpr int ROWS_KC = GEMM_THREADS / TPR_KC;   // KC rows per pass
    static constexpr int TPR_MC = MN / Mfma<T>::VEC;        // threads covering one MC row
    static constexpr int ROWS_MC = GEMM_THREADS / TPR_MC;   // MC rows (k) per pass
    static_assert(MN / ROWS_KC == NVEC && BK / ROWS_MC == NVEC, "NVEC vectors per thread per slab");
    template <bool KC> static constexpr int elems() { return KC ? MN * LDK : BK * LDM; }
};

// Guarded loads of this thread's share of one operand slab (shapes that are not whole tiles or not
// 16-byte aligned).  KC: the operand is stored [mn][k]; MC: it is stored [k][mn].
template <typename T, int WT, bool KC, int DIV = 1>
__device__ __forceinline__ void load_slab_guarded(typename Mfma<T>::Vec (&r)[NV / DIV], const T* __restrict__ base, int64_t ld,
                                                  int64_t mn0, int64_t mn_end, int64_t k0, int64_t k_end, int tid) {
    typedef Slab<T, WT, DIV> S;
    constexpr int VEC = Mfma<T>::VEC;
#pragma unroll
    for (int p = 0; p < NV / DIV; ++p) {
        int64_t mn, k;
        const T* g;
        if (KC) {
            mn = mn0 + tid / S::TPR_KC + S::ROWS_KC * p;
            k = k0 + (tid % S::TPR_KC) * VEC;
            g = base + mn * ld + k;
#pragma unroll
            for (int e = 0; e < VEC; ++e) r[p][e] = (mn < mn_end && k + e < k_end) ? g[e] : (T)0;
        } else {
            k = k0 + tid / S::TPR_MC + S::ROWS_MC * p;
            mn = mn0 + (tid % S::TPR_MC) * VEC;
            g = base + k * ld + mn;
#pragma unroll
            for (int e = 0; e < VEC; ++e) r[p][e] = (k < k_end && mn + e < mn_end) ? g[e] : (T)0;
        }
    }
}

// Unguarded loads of one slab, addressed as a wavefront-uniform base (scalar registers, advanced slab
// by slab) plus a per-thread 32-bit byte offset that never changes.  They are issued as buffer loads so
// that no vector register is ever written to form an address: with per-lane 64-bit pointers the compiler
// advances them with vector adds into registers that loads still in flight are about to fill, and waits
// for those loads (the slab being prefetched) first, which undoes the prefetch.
// A tile that hangs over the edge of the matrix (`valid` < MN rows or columns of it exist) clamps its offsets to
// the last valid row / vector: the threads concerned load duplicates of valid data, which only reach output
// rows or columns that are never stored (row i of the product depends on row i of A alone, column j on column j
// of B alone).  A vector that starts below the edge may run past it, inside the padding of the leading dimension.
// gather_stride > 0 (MC operands only): the MN columns of the tile are four segments of MN / 4 columns that lie
// gather_stride elements apart in memory (the four gate blocks of a fused LSTM weight).
template <typename T, int WT, bool KC, int DIV = 1>
__device__ __forceinline__ void slab_offsets(unsigned (&off)[NV / DIV], int64_t ld, int tid, int valid, int64_t gather_stride = 0) {
    typedef Slab<T, WT, DIV> S;
    constexpr int VEC = Mfma<T>::VEC;
    const int last_vec = ((valid - 1) / VEC) * VEC;
    int col = min((tid % S::TPR_MC) * VEC, last_vec);
    int64_t col_off = col;
    if (!KC && gather_stride > 0) col_off = (col / (S::MN / 4)) * gather_stride + col % (S::MN / 4);
#pragma unroll
    for (int p = 0; p < NV / DIV; ++p)
        off[p] = (unsigned)sizeof(T) * (KC ? (unsigned)(min(tid / S::TPR_KC + S::ROWS_KC * p, valid - 1) * ld + (tid % S::TPR_KC) * VEC)
                                           : (unsigned)((tid / S::TPR_MC + S::ROWS_MC * p) * ld + col_off));
}
template <typename T, int N>
__device__ __forceinline__ void load_slab_fast(typename Mfma<T>::Vec (&r)[N], const T* __restrict__ ubase, const unsigned (&off)[N]) {
    typedef typename Mfma<T>::Vec Vec;
    // A buffer load: descriptor (the base, no bounds in use) in scalar registers, byte offset in one vector register.
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(ubase), 0, -1, 0x00020000);
#pragma unroll
    for (int p = 0; p < N; ++p) r[p] = __builtin_bit_cast(Vec, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off[p], 0, 0));
}

template <typename T, int WT, bool KC, int DIV = 1>
__device__ __forceinline__ void store_slab(T* __restrict__ s, const typename Mfma<T>::Vec (&r)[NV / DIV], int tid) {
    typedef Slab<T, WT, DIV> S;
    typedef typename Mfma<T>::Vec Vec;
    constexpr int VEC = Mfma<T>::VEC;
#pragma unroll
    for (int p = 0; p < NV / DIV; ++p) {
        if (KC) *reinterpret_cast<Vec*>(s + (tid / S::TPR_KC + S::ROWS_KC * p) * S::LDK + (tid % S::TPR_KC) * VEC) = r[p];
        else {
            const int k = tid / S::TPR_MC + S::ROWS_MC * p;
            const int col = ((tid % S::TPR_MC) * VEC + S::mc_shift(k)) & (S::ROTATE_MC ? S::MN - 1 : ~0);
            *reinterpret_cast<Vec*>(s + k * S::LDM + col) = r[p];
        }
    }
}

// The same transfers one 16-byte vector at a time (the main loop issues them between its MFMAs).
template <typename T>
__device__ __forceinline__ typename Mfma<T>::Vec load_vec_fast(const T* __restrict__ ubase, unsigned off) {
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(ubase), 0, -1, 0x00020000);
    return __builtin_bit_cast(typename Mfma<T>::Vec, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, 0));
}
template <typename T, int WT, bool KC, int DIV = 1>
__device__ __forceinline__ void store_vec(T* __restrict__ s, const typename Mfma<T>::Vec& r, int p, int tid) {
    typedef Slab<T, WT, DIV> S;
    typedef typename Mfma<T>::Vec Vec;
    constexpr int VEC = Mfma<T>::VEC;
    if (KC) *reinterpret_cast<Vec*>(s + (tid / S::TPR_KC + S::ROWS_KC * p) * S::LDK + (tid % S::TPR_KC) * VEC) = r;
    else {
        const int k = tid / S::TPR_MC + S::ROWS_MC * p;
        const int col = ((tid % S::TPR_MC) * VEC + S::mc_shift(k)) & (S::ROTATE_MC ? S::MN - 1 : ~0);
        *reinterpret_cast<Vec*>(s + k * S::LDM + col) = r;
    }
}

// Element (mn, k) of a slab in LDS.
template <typename T, int WT, bool KC, int DIV = 1>
__device__ __forceinline__ T slab_at(const T* __restrict__ s, int mn, int k) {
    typedef Slab<T, WT, DIV> S;
    return KC ? s[mn * S::LDK + k] : s[k * S::LDM + ((mn + S::mc_shift(k)) & (S::ROTATE_MC ? S::MN - 1 : ~0))];
}

// Maps the linear workgroup id to an output tile.  Hardware deals consecutive workgroup ids
// round-robin to the 8 XCDs, each with its own L2: ids are first regrouped so that one XCD gets a
// contiguous range of logical tiles, and logical tiles walk the output in bands of GROUP_M tile
// rows, so the tiles resident on one XCD at a time share A row panels and B column panels.
__device__ __forceinline__ void tile_of_workgroup(int pid, int tilesM, int tilesN, int& tm, int& tn) {
    const int nwg = tilesM * tilesN;
    const int per = nwg / NUM_XCD, rem = nwg % NUM_XCD;
    const int xcd = pid % NUM_XCD, slot = pid / NUM_XCD;
    const int lid = xcd < rem ? xcd * (per + 1) + slot : rem * (per + 1) + (xcd - rem) * per + slot;
    const int width = GROUP_M * tilesN;
    const int group = lid / width;
    const int first_m = group * GROUP_M;
    const int gsz = min(tilesM - first_m, GROUP_M);
    const int in_group = lid % width;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
}

constexpr int min_blocks(int) { return 2; }

// Epilogue kinds (template argument EPI).
constexpr int EPI_PLAIN = 0;      // store (or accumulate into) C
constexpr int EPI_ELEMENTWISE = 1;  // bias / pre-activation copy / activation forward / upstream activation backward
constexpr int EPI_TILE_SUM = 2;   // reduce the tile to one double (MatrixMultiplyAndSum forward)
constexpr int EPI_LSTM_FWD = 3;   // gates, cell state and hidden state of one LSTM step (32 x 32 tile gathering 4 gates x 8 units)
constexpr int EPI_LSTM_BWD = 4;   // cell backward of one LSTM step on the recurrent gradient tile

// Workgroup coordinates of a product inside a launch: what blockIdx / gridDim are when the launch holds one product.
struct GridPos {
    unsigned bx, by, bz;  // tile (or rider) index, batch index, split index
    unsigned gy, gz;      // batch count, split count
};

// One workgroup's share of one product (a tile, or the column-sum rider).
// SHORT: thousands of small products whose K is a slab or less (the attention products of a windowed block,
// K = 32 or 49).  Software pipelining has nothing to work with there, so the kernel keeps one LDS stage instead
// of two and no prefetch registers: more workgroups share a compute unit and overlap one another's loads,
// products and stores.  It multiplies only the k steps that the last slab has.
// LDS of one workgroup of gemm_tile: the slab stages ([stage][A slab | B slab]), reused by the epilogues.
template <typename T, int WT, bool A_KC, bool B_KC, bool SHORT = false, int DIV = 1>
constexpr int gemm_lds_elems() {
    return (SHORT ? 1 : 2) * (Slab<T, WT, DIV>::template elems<A_KC>() + Slab<T, WT, DIV>::template elems<B_KC>());
}

// `lds`: gemm_lds_elems<...>() elements of 16-byte aligned LDS that the kernel provides (a kernel that holds two
// products gives both the same block).
template <typename T, int WT, bool A_KC, bool B_KC, bool EDGE, int EPI, bool SHORT = false, int DIV = 1>
__device__ __forceinline__ void gemm_tile(const GemmArgs<T>& p, const int tilesM, const int tilesN, const GridPos g_, T* __restrict__ lds) {
    typedef Mfma<T> MF;
    typedef Slab<T, WT, DIV> S;
    typedef typename MF::Acc Acc;
    typedef typename MF::Vec Vec;
    constexpr int BK = S::BK;
    constexpr int BM = 32 * WT, BN = 32 * WT;  // output tile
    constexpr int WS = 16 * WT;                // edge of one wavefront's share
    constexpr int WTM = WT, WTN = WT;
    constexpr int SA = S::template elems<A_KC>(), SB = S::template elems<B_KC>();

    static_assert(!SHORT || (EDGE && EPI == EPI_PLAIN), "the single-stage kernel is guarded and stores plainly");
    T (*smem)[SA + SB] = reinterpret_cast<T (*)[SA + SB]>(lds);  // [stage][A slab | B slab]

    // Workgroups beyond the tiles carry a column sum that rides along with this launch.
    if (g_.bx >= (unsigned)(tilesM * tilesN)) {
        if (g_.by == 0 && g_.bz == 0)
            colsum_block<T, T>(p.colsum_src, p.colsum_dst, p.colsum_cols, 0, p.colsum_rows, g_.bx - tilesM * tilesN,
                               reinterpret_cast<double*>(&smem[0][0]));
        return;
    }
    int tm, tn;
    tile_of_workgroup(g_.bx, tilesM, tilesN, tm, tn);
    const int64_t row0 = (int64_t)tm * BM, col0 = (int64_t)tn * BN;
    const int batch = g_.by;
    const int b_outer = p.batch_inner > 1 ? batch / p.batch_inner : batch;
    const int b_inner = p.batch_inner > 1 ? batch - b_outer * p.batch_inner : 0;
    const T* __restrict__ A = p.A + b_outer * p.strideA + b_inner * p.istrideA;
    const T* __restrict__ B = p.B + b_outer * p.strideB + b_inner * p.istrideB;
    // A product split along K: this workgroup reduces [kb, kb + K) and writes its own M x N partial result.
    int64_t K = p.K;
    if (g_.gz > 1) {
        const int64_t kb = (int64_t)g_.bz * p.ksplit;
        K = min(p.ksplit, p.K - kb);
        A += (int64_t)g_.bz * p.zstrideA;
        B += (int64_t)g_.bz * p.zstrideB;
    }

    // (not const: they are formed again after the K loop, see there)
    int tid = threadIdx.x;
    const int wave_scalar = __builtin_amdgcn_readfirstlane(tid >> 6);
    int lane = tid & 63, wave = tid >> 6;
    int wm = wave >> 1, wn = wave & 1;
    int li = lane & 15, g = lane >> 4;

    Acc acc[WTM][WTN];
#pragma unroll
    for (int x = 0; x < WTM; ++x)
#pragma unroll
        for (int y = 0; y < WTN; ++y)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[x][y][r] = (T)0;
    // Float products of a long K: a single chain of MFMA accumulations rounds every step at the magnitude of the
    // running sum, and at K of several thousand that noise reaches the 1e-5 parity bar by itself.  The accumulators
    // are therefore folded into a second set every FOLD_K of the reduction (two-level summation: chains of at most
    // FOLD_K / 4 steps, then one addition per fold).  Products of K <= FOLD_K give the bits they gave without it.
    constexpr int FOLD_K = PRAD_GEMM_FOLD_K;
    // (the single-stage and half-depth kernels only take K <= FOLD_K; the LSTM step kernels reduce at most 4 * hidden)
    constexpr bool FOLD = FOLD_K > 0 && sizeof(T) == 4 && !SHORT && DIV == 1 && EPI != EPI_LSTM_FWD && EPI != EPI_LSTM_BWD;
    constexpr int FOLD_SLABS = FOLD ? FOLD_K / BK : 2;
    static_assert(!FOLD || (FOLD_SLABS >= 2 && (FOLD_SLABS & (FOLD_SLABS - 1)) == 0), "folds fall on even slab counts");
    Acc acc2[FOLD ? WTM : 1][FOLD ? WTN : 1];
    if (FOLD) {
#pragma unroll
        for (int x = 0; x < WTM; ++x)
#pragma unroll
            for (int y = 0; y < WTN; ++y)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc2[x][y][r] = (T)0;
    }
    auto fold = [&] {
        if (FOLD) {
#pragma unroll
            for (int x = 0; x < WTM; ++x)
#pragma unroll
                for (int y = 0; y < WTN; ++y)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        acc2[x][y][r] = acc2[x][y][r] + acc[x][y][r];
                        acc[x][y][r] = (T)0;
                    }
        }
    };

    // Unguarded kernels run the whole slabs with vector loads and finish a ragged end of K (784 = 12 x 64 + 16)
    // with one guarded slab; guarded kernels treat every slab alike.
    const int ntiles = EDGE ? (int)((K + BK - 1) / BK) : (int)(K / BK);

    // One slab of MFMAs from the LDS stage at `st`.
    auto compute = [&](const T* __restrict__ st) {
        const T* __restrict__ sA = st;
        const T* __restrict__ sB = st + SA;
        // While a wavefront multiplies it outranks its SIMD's other wavefront (which is then loading or waiting at a
        // barrier) at instruction issue: measured +2.3 % at N = 4096 in double.
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int s = 0; s < BK / 4; ++s) {
            const int k = 4 * s + g;
            T a[WTM], b[WTN];
#pragma unroll
            for (int x = 0; x < WTM; ++x) a[x] = slab_at<T, WT, A_KC, DIV>(sA, wm * WS + x * 16 + li, k);
#pragma unroll
            for (int y = 0; y < WTN; ++y) b[y] = slab_at<T, WT, B_KC, DIV>(sB, wn * WS + y * 16 + li, k);
#pragma unroll
            for (int x = 0; x < WTM; ++x)
#pragma unroll
                for (int y = 0; y < WTN; ++y) acc[x][y] = MF::run(a[x], b[y], acc[x][y]);
        }
        __builtin_amdgcn_s_setprio(0);
    };

    // The same slab of MFMAs with the workgroup's other work issued in their shadow.  A wavefront that issues an MFMA
    // is free to issue other instructions while the matrix core works on it (16 to 64 cycles), but the next MFMA has
    // to wait for the core; so every MFMA is followed by at most a few of: the LDS reads of the next k step's
    // fragments (read one step ahead into a second set of registers), and `op(o)`, o in [0, NOPS) - the caller's
    // transfers for the slabs ahead (one 16-byte vector each: registers -> the other LDS stage, memory -> registers).
    // Issued as blocks before and after the MFMAs of a slab, those transfers and the wait for the first fragments
    // left the matrix core idle for a third of the time of a workgroup that has its compute unit to itself.
    // The MFMAs run in the same order on the same operands as in `compute`: same bits.
    constexpr int NM = WTM * WTN, NR = WTM + WTN, KSTEPS = BK / 4, SLOTS = KSTEPS * NM;
    auto compute_mix = [&](const T* __restrict__ st, auto&& op, auto nops_) {
        constexpr int NOPS = decltype(nops_)::value;
        const T* __restrict__ sA = st;
        const T* __restrict__ sB = st + SA;
        T a[2][WTM], b[2][WTN];
        auto read = [&](int s, int r) {
            const int k = 4 * s + g;
            if (r < WTM) a[s & 1][r] = slab_at<T, WT, A_KC, DIV>(sA, wm * WS + r * 16 + li, k);
            else b[s & 1][r - WTM] = slab_at<T, WT, B_KC, DIV>(sB, wn * WS + (r - WTM) * 16 + li, k);
        };
#pragma unroll
        for (int r = 0; r < NR; ++r) read(0, r);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                const int x = m / WTN, y = m % WTN;
                acc[x][y] = MF::run(a[s & 1][x], b[s & 1][y], acc[x][y]);
                if (s + 1 < KSTEPS) {
#pragma unroll
                    for (int r = m * NR / NM; r < (m + 1) * NR / NM; ++r) read(s + 1, r);
                }
                const int q = s * NM + m;
#pragma unroll
                for (int o = q * NOPS / SLOTS; o < (q + 1) * NOPS / SLOTS; ++o) op(o);
                __builtin_amdgcn_sched_barrier(0);  // (the scheduler would gather the transfers into blocks again)
            }
        }
        __builtin_amdgcn_s_setprio(0);
    };

    if (SHORT) {
        // One LDS stage and no prefetch: the loads of a slab are hidden by the other workgroups of the compute unit.
        Vec ra[S::NVEC], rb[S::NVEC];
        const int nslabs = (int)((K + BK - 1) / BK);  // one where the launch rules send products here
        for (int kt = 0; kt < nslabs; ++kt) {
            const int64_t k0 = (int64_t)kt * BK;
            load_slab_guarded<T, WT, A_KC, DIV>(ra, A, p.lda, row0, p.M, k0, K, tid);
            load_slab_guarded<T, WT, B_KC, DIV>(rb, B, p.ldb, col0, p.N, k0, K, tid);
            if (kt > 0) __syncthreads();  // every wavefront is done with the slab before
            store_slab<T, WT, A_KC, DIV>(smem[0], ra, tid);
            store_slab<T, WT, B_KC, DIV>(smem[0] + SA, rb, tid);
            __syncthreads();
            const T* __restrict__ sA = smem[0];
            const T* __restrict__ sB = smem[0] + SA;
            const int ksteps = (int)((min((int64_t)BK, K - k0) + 3) / 4);  // the slab is zero beyond K
#pragma unroll 2
            for (int s = 0; s < ksteps; ++s) {
                const int k = 4 * s + g;
                T a[WTM], b[WTN];
#pragma unroll
                for (int x = 0; x < WTM; ++x) a[x] = slab_at<T, WT, A_KC, DIV>(sA, wm * WS + x * 16 + li, k);
#pragma unroll
                for (int y = 0; y < WTN; ++y) b[y] = slab_at<T, WT, B_KC, DIV>(sB, wn * WS + y * 16 + li, k);
#pragma unroll
                for (int x = 0; x < WTM; ++x)
#pragma unroll
                    for (int y = 0; y < WTN; ++y) acc[x][y] = MF::run(a[x], b[y], acc[x][y]);
            }
        }
    } else if (!EDGE) {
        // Two register sets: while slab t is multiplied out of LDS, slab t+1 waits in one set and the loads
        // of slab t+2 are issued into the other, so a global load has two slabs of MFMAs to arrive.  The loop
        // is unrolled by two so that the sets are named statically.
        Vec ra0[S::NVEC], rb0[S::NVEC], ra1[S::NVEC], rb1[S::NVEC];
        unsigned offa[S::NVEC], offb[S::NVEC];
        slab_offsets<T, WT, A_KC, DIV>(offa, p.lda, tid, (int)min((int64_t)BM, p.M - row0));
        constexpr bool GATHER = EPI == EPI_LSTM_FWD;  // B columns: 4 gate segments of BN / 4 hidden units each
        if (GATHER) slab_offsets<T, WT, B_KC, DIV>(offb, p.ldb, tid, BN, p.lstm_hidden);
        else slab_offsets<T, WT, B_KC, DIV>(offb, p.ldb, tid, (int)min((int64_t)BN, p.N - col0));
        // uniform bases of slab 0 and their per-slab strides
        const T* __restrict__ ua = A + (A_KC ? row0 * p.lda : row0);
        const T* __restrict__ ub = B + (GATHER ? (int64_t)tn * (BN / 4) : (B_KC ? col0 * p.ldb : col0));
        const int64_t stepa = A_KC ? (int64_t)BK : (int64_t)BK * p.lda;
        const int64_t stepb = B_KC ? (int64_t)BK : (int64_t)BK * p.ldb;
        // The loads inside the loop stand in straight-line code: at a branch around a load the compiler loses count
        // of the loads in flight and from then on waits for all of them before every use, which undoes the prefetch.
        // The loop therefore runs while both slabs it fetches exist, and the last one to three slabs drain after it.
        if (ntiles > 0) {
            load_slab_fast<T>(ra0, ua, offa);
            load_slab_fast<T>(rb0, ub, offb);
            load_slab_fast<T>(ra1, ua + min(1, ntiles - 1) * stepa, offa);  // (the only slab twice if K holds just one)
            load_slab_fast<T>(rb1, ub + min(1, ntiles - 1) * stepb, offb);
            store_slab<T, WT, A_KC, DIV>(smem[0], ra0, tid);
            store_slab<T, WT, B_KC, DIV>(smem[0] + SA, rb0, tid);
            __syncthreads();
            int kt = 0;
            constexpr int NV_ = S::NVEC;
            constexpr bool MIX = WT <= PRAD_GEMM_MIX_WT;
            constexpr bool MIX_DRAIN = MIX && WT <= 2;  // (the 128 x 128 kernels have no registers to spare for the extra code paths: hundreds of spills)
            for (; kt + 3 < ntiles; kt += 2) {
                // LDS stage 0 holds slab kt, set 1 holds slab kt+1 (in flight), set 0 is free.
                if (MIX) {
                    // even o: vector o/2 of slab kt+1, registers -> stage 1 (free since the barrier); odd o: vector o/2 of slab kt+2, memory -> set 0
                    const T* __restrict__ na = ua + (kt + 2) * stepa;
                    const T* __restrict__ nb = ub + (kt + 2) * stepb;
                    compute_mix(smem[0], [&](int o) {
                        const int j = o >> 1;
                        if (o & 1) { if (j < NV_) ra0[j] = load_vec_fast<T>(na, offa[j]); else rb0[j - NV_] = load_vec_fast<T>(nb, offb[j - NV_]); }
                        else { if (j < NV_) store_vec<T, WT, A_KC, DIV>(smem[1], ra1[j], j, tid); else store_vec<T, WT, B_KC, DIV>(smem[1] + SA, rb1[j - NV_], j - NV_, tid); }
                    }, std::integral_constant<int, 4 * NV_>{});
                    __syncthreads();
                    const T* __restrict__ ma = ua + (kt + 3) * stepa;
                    const T* __restrict__ mb = ub + (kt + 3) * stepb;
                    compute_mix(smem[1], [&](int o) {
                        const int j = o >> 1;
                        if (o & 1) { if (j < NV_) ra1[j] = load_vec_fast<T>(ma, offa[j]); else rb1[j - NV_] = load_vec_fast<T>(mb, offb[j - NV_]); }
                        else { if (j < NV_) store_vec<T, WT, A_KC, DIV>(smem[0], ra0[j], j, tid); else store_vec<T, WT, B_KC, DIV>(smem[0] + SA, rb0[j - NV_], j - NV_, tid); }
                    }, std::integral_constant<int, 4 * NV_>{});
                    if (FOLD && ((kt + 2) & (FOLD_SLABS - 1)) == 0) fold();
                    __syncthreads();
                    continue;
                }
                load_slab_fast<T>(ra0, ua + (kt + 2) * stepa, offa);
                load_slab_fast<T>(rb0, ub + (kt + 2) * stepb, offb);
                compute(smem[0]);
                store_slab<T, WT, A_KC, DIV>(smem[1], ra1, tid);
                store_slab<T, WT, B_KC, DIV>(smem[1] + SA, rb1, tid);
                __syncthreads();
                load_slab_fast<T>(ra1, ua + (kt + 3) * stepa, offa);
                load_slab_fast<T>(rb1, ub + (kt + 3) * stepb, offb);
                compute(smem[1]);
                if (FOLD && ((kt + 2) & (FOLD_SLABS - 1)) == 0) fold();
                store_slab<T, WT, A_KC, DIV>(smem[0], ra0, tid);
                store_slab<T, WT, B_KC, DIV>(smem[0] + SA, rb0, tid);
                __syncthreads();
            }
            // left: slab kt in stage 0, slab kt+1 (if any) in set 1, slab kt+2 (if any) still to be fetched
            if (MIX_DRAIN && kt + 1 < ntiles) {
                auto stores_1 = [&](int j) {  // slab kt+1: set 1 -> stage 1
                    if (j < NV_) store_vec<T, WT, A_KC, DIV>(smem[1], ra1[j], j, tid); else store_vec<T, WT, B_KC, DIV>(smem[1] + SA, rb1[j - NV_], j - NV_, tid);
                };
                if (kt + 2 < ntiles) {
                    const T* __restrict__ na = ua + (kt + 2) * stepa;
                    const T* __restrict__ nb = ub + (kt + 2) * stepb;
                    compute_mix(smem[0], [&](int o) {
                        const int j = o >> 1;
                        if (o & 1) { if (j < NV_) ra0[j] = load_vec_fast<T>(na, offa[j]); else rb0[j - NV_] = load_vec_fast<T>(nb, offb[j - NV_]); }
                        else stores_1(j);
                    }, std::integral_constant<int, 4 * NV_>{});
                    __syncthreads();
                    compute_mix(smem[1], [&](int j) {  // slab kt+2: set 0 -> stage 0
                        if (j < NV_) store_vec<T, WT, A_KC, DIV>(smem[0], ra0[j], j, tid); else store_vec<T, WT, B_KC, DIV>(smem[0] + SA, rb0[j - NV_], j - NV_, tid);
                    }, std::integral_constant<int, 2 * NV_>{});
                    __syncthreads();
                    compute_mix(smem[0], [](int) {}, std::integral_constant<int, 0>{});
                } else {
                    compute_mix(smem[0], stores_1, std::integral_constant<int, 2 * NV_>{});
                    __syncthreads();
                    compute_mix(smem[1], [](int) {}, std::integral_constant<int, 0>{});
                }
            } else {
            if (kt + 2 < ntiles) {
                load_slab_fast<T>(ra0, ua + (kt + 2) * stepa, offa);
                load_slab_fast<T>(rb0, ub + (kt + 2) * stepb, offb);
            }
            compute(smem[0]);
            if (kt + 1 < ntiles) {
                store_slab<T, WT, A_KC, DIV>(smem[1], ra1, tid);
                store_slab<T, WT, B_KC, DIV>(smem[1] + SA, rb1, tid);
                __syncthreads();
                compute(smem[1]);
            }
            if (kt + 2 < ntiles) {
                store_slab<T, WT, A_KC, DIV>(smem[0], ra0, tid);
                store_slab<T, WT, B_KC, DIV>(smem[0] + SA, rb0, tid);
                __syncthreads();
                compute(smem[0]);
            }
            }
        }
        if ((int64_t)ntiles * BK < K) {    // ragged end of K: one guarded slab through stage 1
            load_slab_guarded<T, WT, A_KC, DIV>(ra1, A, p.lda, row0, p.M, (int64_t)ntiles * BK, K, tid);
            load_slab_guarded<T, WT, B_KC, DIV>(rb1, B, p.ldb, col0, p.N, (int64_t)ntiles * BK, K, tid);
            __syncthreads();  // every wavefront is done with the last whole slab, whichever stage held it
            store_slab<T, WT, A_KC, DIV>(smem[1], ra1, tid);
            store_slab<T, WT, B_KC, DIV>(smem[1] + SA, rb1, tid);
            __syncthreads();
            compute(smem[1]);
        }
    } else {
        Vec ra[S::NVEC], rb[S::NVEC];
        load_slab_guarded<T, WT, A_KC, DIV>(ra, A, p.lda, row0, p.M, 0, K, tid);
        load_slab_guarded<T, WT, B_KC, DIV>(rb, B, p.ldb, col0, p.N, 0, K, tid);
        store_slab<T, WT, A_KC, DIV>(smem[0], ra, tid);
        store_slab<T, WT, B_KC, DIV>(smem[0] + SA, rb, tid);
        __syncthreads();
        int cur = 0;
        for (int kt = 0; kt < ntiles; ++kt) {
            const bool more = kt + 1 < ntiles;
            if (more) {
                load_slab_guarded<T, WT, A_KC, DIV>(ra, A, p.lda, row0, p.M, (int64_t)(kt + 1) * BK, K, tid);
                load_slab_guarded<T, WT, B_KC, DIV>(rb, B, p.ldb, col0, p.N, (int64_t)(kt + 1) * BK, K, tid);
            }
            compute(smem[cur]);
            if (FOLD && ((kt + 1) & (FOLD_SLABS - 1)) == 0) fold();
            if (more) {
                store_slab<T, WT, A_KC, DIV>(smem[cur ^ 1], ra, tid);
                store_slab<T, WT, B_KC, DIV>(smem[cur ^ 1] + SA, rb, tid);
            }
            __syncthreads();
            cur ^= 1;
        }
    }

    // The epilogues use the thread's coordinates again.  Kept alive across the K loop, where every register is taken,
    // they were spilled before it (five dwords per lane, 5 MiB of scratch writes per launch of the 128 x 128 kernel in
    // double); formed anew from a thread index the compiler cannot tie to the one above, they cost a few instructions.
    // (Each epilogue path forms them for itself: held from here across the other paths they were spilled again.)
    // (The lane comes from the hardware's lane count and the wavefront's number from a scalar register: the thread index
    // itself would have to be kept, which is a spilled register as well.)
    auto coordinates = [&] {
        unsigned all = ~0u;
        asm volatile("" : "+s"(all));  // (opaque, so that the count is taken anew at every call instead of being kept)
        const int l = (int)__builtin_amdgcn_mbcnt_hi(all, __builtin_amdgcn_mbcnt_lo(all, 0u));
        lane = l; wave = wave_scalar; tid = 64 * wave + lane; wm = wave >> 1; wn = wave & 1; li = lane & 15; g = lane >> 4;
    };
    coordinates();
    if (FOLD) {
#pragma unroll
        for (int x = 0; x < WTM; ++x)
#pragma unroll
            for (int y = 0; y < WTN; ++y)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[x][y][r] = acc2[x][y][r] + acc[x][y][r];
    }

    // ---- epilogue ------------------------------------------------------------------------
    if (EPI == EPI_TILE_SUM) {
        // Sum of the whole tile (rows/columns past M, N hold exact zeros).
        double s = 0.0;
#pragma unroll
        for (int x = 0; x < WTM; ++x)
#pragma unroll
            for (int y = 0; y < WTN; ++y)
#pragma unroll
                for (int r = 0; r < 4; ++r) s += (double)acc[x][y][r];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) s += __shfl_down(s, off, 64);
        __syncthreads();  // every wavefront is done with the slab stages
        double* red = reinterpret_cast<double*>(&smem[0][0]);
        if (lane == 0) red[wave] = s;
        __syncthreads();
        if (tid == 0)
            p.tile_sums[(int64_t)batch * tilesM * tilesN + (int64_t)tm * tilesN + tn] = (red[0] + red[1]) + (red[2] + red[3]);
        return;
    }

    if (EPI != EPI_TILE_SUM && p.split_counters != nullptr && g_.gz > 1) {
        coordinates();
        // Several workgroups share this tile, a K range each.  Every one parks its partial tile in the workspace
        // and counts its arrival; the one that arrives last adds the partial tiles in split order (its own
        // included, read back like the others, so that the sum does not depend on who arrives last) and goes on
        // to the epilogue.  No workgroup waits for another.  The partial tiles travel as device-coherent stores and
        // loads (written through to memory, read past the per-XCD caches): a device-scope fence would write back and
        // invalidate the whole L2 and evict the operand panels of every workgroup nearby.  What orders them:
        //   writer: every wavefront waits for its own parked stores to be acknowledged (vmcnt(0): a write-through
        //           store is acknowledged once it is in memory), then the workgroup barrier, then thread 0's
        //           device-scope atomic add on the tile's counter.  The workgroup barrier alone does not wait for
        //           outstanding vector stores.
        //   reader: the last arriver sees the count (the atomic's return value, through LDS and a barrier) before it
        //           issues its device-coherent loads, which therefore find every other workgroup's tile in memory.
        const int64_t mn = p.M * p.N;
        const int splits = (int)g_.gz;
        T* __restrict__ mine = p.split_ws + ((int64_t)g_.bz * g_.gy + batch) * mn;
#pragma unroll
        for (int x = 0; x < WTM; ++x)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t i = row0 + wm * WS + x * 16 + MF::row(r, g);
#pragma unroll
                for (int y = 0; y < WTN; ++y) {
                    const int64_t j = col0 + wn * WS + y * 16 + li;
                    if (i >= p.M || j >= p.N) continue;
                    __hip_atomic_store(&mine[i * p.N + j], acc[x][y][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // compiler: the stores stay above the wait
        __builtin_amdgcn_s_waitcnt(0x0F70);                      // vmcnt(0), other counters untouched
        __syncthreads();
        __shared__ unsigned arrived;
        if (tid == 0) {
            unsigned* c = p.split_counters + (int64_t)batch * tilesM * tilesN + (int64_t)tm * tilesN + tn;
            arrived = atomicAdd(c, 1u);
            if (arrived == (unsigned)splits - 1u) *c = 0u;  // left zeroed for the next launch
        }
        __syncthreads();
        if (arrived != (unsigned)splits - 1u) return;
        // Partial tiles of ZU splits are fetched together, 16 rows of the wavefront's share at a time, so that
        // enough loads are in flight without holding a second copy of the whole tile in registers.
        constexpr int ZU = WT == 4 ? 1 : (WT == 2 ? 4 : 8);
        for (int z0 = 0; z0 < splits; z0 += ZU) {
#pragma unroll
            for (int x = 0; x < WTM; ++x) {
                T part[ZU][WTN][4];
#pragma unroll
                for (int u = 0; u < ZU; ++u) {
                    if (z0 + u >= splits) break;
                    const T* other = p.split_ws + ((int64_t)(z0 + u) * g_.gy + batch) * mn;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int64_t i = row0 + wm * WS + x * 16 + MF::row(r, g);
#pragma unroll
                        for (int y = 0; y < WTN; ++y) {
                            const int64_t j = col0 + wn * WS + y * 16 + li;
                            part[u][y][r] = (i >= p.M || j >= p.N)
                                                ? (T)0
                                                : __hip_atomic_load(&other[i * p.N + j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < ZU; ++u) {
                    if (z0 + u >= splits) break;
#pragma unroll
                    for (int y = 0; y < WTN; ++y)
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[x][y][r] = (z0 + u == 0) ? part[u][y][r] : acc[x][y][r] + part[u][y][r];
                }
            }
        }
    }

    if (WT == 4 && EPI != EPI_TILE_SUM && p.shared_splits > 1 && g_.gz > 1) {
        coordinates();
        // One of the workgroups that share a tile of an otherwise unsplit launch: its partial tile goes to the workspace
        // as a plain 128 x 128 row-major block (tile by tile, split by split); shared_reduce_kernel adds the blocks of a
        // tile in split order and applies the epilogue.
        T* __restrict__ mine = p.split_ws + ((int64_t)g_.bx * g_.gz + g_.bz) * (BM * BN);
#pragma unroll
        for (int x = 0; x < WTM; ++x)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int il = wm * WS + x * 16 + MF::row(r, g);
#pragma unroll
                for (int y = 0; y < WTN; ++y) mine[il * BN + wn * WS + y * 16 + li] = acc[x][y][r];
            }
        return;
    }

    if (EPI == EPI_LSTM_FWD) {
        // The tile holds h_{t-1} . W_h for 32 rows and, column block q of 8, gate q of hidden units [8 tn, 8 tn + 8).
        // It goes through LDS so that one thread gets the four gates of one (row, unit); then the arithmetic of
        // lstm_cell_fwd_kernel, statement for statement.
        static_assert(EPI != EPI_LSTM_FWD || WT == 1, "the gate gather is laid out for the 32 x 32 tile");
        constexpr int LDT = BN + 1;
        __syncthreads();  // every wavefront is done with the slab stages
        T* __restrict__ stage = &smem[0][0];
#pragma unroll
        for (int r = 0; r < 4; ++r) stage[(wm * WS + MF::row(r, g)) * LDT + wn * WS + li] = acc[0][0][r];
        __syncthreads();
        const int row = tid / 8, jj = tid % 8;
        const int64_t i = row0 + row, H = p.lstm_hidden, j = (int64_t)tn * 8 + jj;
        if (i < p.M) {
            T* __restrict__ gr = p.C + i * p.ldc;  // pre-activations (input projection + bias) in, activated gates out
            const T* __restrict__ st = stage + row * LDT + jj;
            const T i_ = act_forward<T>(ACT_SIGMOID, gr[j] + st[0], (T)0);
            const T f_ = act_forward<T>(ACT_SIGMOID, gr[H + j] + st[8], (T)0);
            const T g_ = act_forward<T>(ACT_TANH, gr[2 * H + j] + st[16], (T)0);
            const T o_ = act_forward<T>(ACT_SIGMOID, gr[3 * H + j] + st[24], (T)0);
            gr[j] = i_; gr[H + j] = f_; gr[2 * H + j] = g_; gr[3 * H + j] = o_;
            const int64_t idx = i * H + j;
            const T cn = (f_ * p.lstm_c_prev[idx]) + (i_ * g_);
            const T tc = act_forward<T>(ACT_TANH, cn, (T)0);
            p.lstm_c[idx] = cn;
            p.lstm_tanh_c[idx] = tc;
            p.lstm_h[idx] = o_ * tc;
        }
        return;
    }

    if (EPI == EPI_LSTM_BWD) {
        // The tile is (dG_{t+1} . W_h^T), the recurrent part of dh, for 32 rows x 32 hidden units.  It goes through
        // LDS so that a thread takes four elements of consecutive rows with all their loads in flight at once; then
        // the arithmetic of lstm_cell_bwd_kernel, statement for statement.
        static_assert(EPI != EPI_LSTM_BWD || WT == 1, "laid out for the 32 x 32 tile");
        constexpr int LDT = BN + 1;
        __syncthreads();  // every wavefront is done with the slab stages
        T* __restrict__ stage = &smem[0][0];
#pragma unroll
        for (int r = 0; r < 4; ++r) stage[(wm * WS + MF::row(r, g)) * LDT + wn * WS + li] = acc[0][0][r];
        __syncthreads();
        const int64_t H = p.lstm_hidden;
        const int cc = tid & 31, rbase = tid >> 5;  // rows rbase, rbase + 8, rbase + 16, rbase + 24
        const int64_t j = col0 + cc;
        T i_[4], f_[4], g_[4], o_[4], tc[4], dhl[4], dci[4], cp[4];
        bool ok[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t i = row0 + rbase + 8 * u;
            ok[u] = i < p.M && j < H;
            if (ok[u]) {
                const T* __restrict__ gt = p.lstm_gates + i * 4 * H;
                const int64_t idx = i * H + j;
                i_[u] = gt[j]; f_[u] = gt[H + j]; g_[u] = gt[2 * H + j]; o_[u] = gt[3 * H + j];
                tc[u] = p.lstm_tanh_c_in[idx];
                dhl[u] = p.lstm_dh_loss[idx];
                dci[u] = p.lstm_dc_in != nullptr ? p.lstm_dc_in[idx] : (T)0;
                cp[u] = p.lstm_c_prev[idx];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (!ok[u]) continue;
            const int64_t i = row0 + rbase + 8 * u, idx = i * H + j;
            T* __restrict__ dg = p.lstm_dG + i * 4 * H;
            const T dh = dhl[u] + stage[(rbase + 8 * u) * LDT + cc];
            const T d_o = dh * tc[u];
            T dc = (dh * o_[u]) * act_derivative<T>(ACT_TANH, tc[u], (T)0);
            if (p.lstm_dc_in != nullptr) dc = dc + dci[u];
            const T d_i = dc * g_[u], d_g = dc * i_[u], d_f = dc * cp[u];
            p.lstm_dc_prev[idx] = dc * f_[u];
            dg[j] = d_i * act_derivative<T>(ACT_SIGMOID, i_[u], (T)0);
            dg[H + j] = d_f * act_derivative<T>(ACT_SIGMOID, f_[u], (T)0);
            dg[2 * H + j] = d_g * act_derivative<T>(ACT_TANH, g_[u], (T)0);
            dg[3 * H + j] = d_o * act_derivative<T>(ACT_SIGMOID, o_[u], (T)0);
        }
        return;
    }

    T* __restrict__ C = p.C + b_outer * p.strideC + b_inner * p.istrideC +
                        ((g_.gz > 1 && p.split_counters == nullptr) ? (int64_t)g_.bz * g_.gy * p.strideC : 0);
    if (EPI == EPI_ELEMENTWISE) {
        coordinates();
        // The accumulators go through LDS, 16 rows of the wavefront's share at a time, and are read back
        // row-major: the elementwise arithmetic (which includes exp/tanh code) then sits in one runtime loop
        // instead of being inlined into 64 unrolled stores, and every global access covers whole rows.
        constexpr int LDW = WS + 4;
        __syncthreads();  // every wavefront is done with the slab stages
        T* __restrict__ stage = &smem[0][0] + wave * (16 * LDW);
        T* __restrict__ side = &smem[0][0] + (4 + wave) * (16 * LDW);  // the values act' is taken of, fetched ahead
        static_assert(EPI != EPI_ELEMENTWISE || 8 * 16 * LDW <= 2 * (SA + SB), "both staging areas fit into the slab stages");
        constexpr int VEC = MF::VEC;
        auto vec_aligned = [](const void* q, int64_t ld) { return q == nullptr || (reinterpret_cast<uintptr_t>(q) % 16 == 0 && ld % VEC == 0); };
        const bool vec_ok = p.N % VEC == 0 && vec_aligned(C, p.ldc) && vec_aligned(p.Z, p.ldz) && vec_aligned(p.act_src, p.ld_act) &&
                            vec_aligned(p.bias, VEC);
        // Each wavefront stages, reads back and stores its own share, so the passes are ordered inside the wavefront
        // only: a workgroup barrier here would also make every pass wait for the global stores of the pass before.
        auto wave_sync = [] {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        };
        // The values act' is taken of, for one pass: all its loads are issued together, and a pass ahead, so that
        // they are in flight during the arithmetic and the stores of the pass before.
        constexpr int SRC_N = 16 * WS / 64;
        T src[SRC_N];
        auto fetch_src = [&](int x) {
#pragma unroll
            for (int it = 0; it < SRC_N; ++it) {
                const int idx = lane + 64 * it, rr = idx / WS, c = idx % WS;
                const int64_t i = row0 + wm * WS + x * 16 + rr, j = col0 + wn * WS + c;
                src[it] = (i < p.M && j < p.N) ? p.act_src[i * p.ld_act + j] : (T)0;
            }
        };
        if (p.act_bwd != ACT_NONE) fetch_src(0);
#pragma unroll
        for (int x = 0; x < WTM; ++x) {
#pragma unroll
            for (int y = 0; y < WTN; ++y)
#pragma unroll
                for (int r = 0; r < 4; ++r) stage[MF::row(r, g) * LDW + y * 16 + li] = acc[x][y][r];
            if (p.act_bwd != ACT_NONE) {
                // each lane parks what it fetched in LDS at the position it was fetched for
#pragma unroll
                for (int it = 0; it < SRC_N; ++it) {
                    const int idx = lane + 64 * it;
                    side[(idx / WS) * LDW + idx % WS] = src[it];
                }
                if (x + 1 < WTM) fetch_src(x + 1);
            }
            wave_sync();
            if (vec_ok) {
                // 16 bytes per lane and access: whole rows of the tile leave in 1 KiB pieces.
#pragma unroll 1
                for (int idx = lane; idx < 16 * WS / VEC; idx += 64) {
                    const int rr = idx / (WS / VEC), c = (idx % (WS / VEC)) * VEC;
                    const int64_t i = row0 + wm * WS + x * 16 + rr;
                    const int64_t j = col0 + wn * WS + c;
                    if (i >= p.M || j >= p.N) continue;  // N is a multiple of VEC here: a vector is inside or outside
                    Vec v = *reinterpret_cast<const Vec*>(stage + rr * LDW + c);
                    if (p.bias != nullptr) {
                        const Vec b = *reinterpret_cast<const Vec*>(p.bias + j);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) v[e] = v[e] + b[e];
                    }
                    if (p.Z != nullptr) *reinterpret_cast<Vec*>(p.Z + i * p.ldz + j) = v;
                    if (p.act_fwd != ACT_NONE) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) v[e] = act_forward<T>(p.act_fwd, v[e], p.alpha);
                    }
                    if (p.act_bwd != ACT_NONE) {
                        const Vec sv = *reinterpret_cast<const Vec*>(side + rr * LDW + c);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) v[e] = v[e] * act_derivative<T>(p.act_bwd, sv[e], p.alpha);
                    }
                    Vec* c_out = reinterpret_cast<Vec*>(C + i * p.ldc + j);
                    if (p.accumulate) {
                        const Vec old = *c_out;
#pragma unroll
                        for (int e = 0; e < VEC; ++e) v[e] = old[e] + v[e];
                    }
                    *c_out = v;
                }
                wave_sync();
                continue;
            }
#pragma unroll 1
            for (int idx = lane; idx < 16 * WS; idx += 64) {
                const int rr = idx / WS, c = idx % WS;
                const int64_t i = row0 + wm * WS + x * 16 + rr;
                const int64_t j = col0 + wn * WS + c;
                if (i >= p.M || j >= p.N) continue;
                T v = stage[rr * LDW + c];
                if (p.bias != nullptr) v = v + p.bias[j];
                if (p.Z != nullptr) p.Z[i * p.ldz + j] = v;
                if (p.act_fwd != ACT_NONE) v = act_forward<T>(p.act_fwd, v, p.alpha);
                if (p.act_bwd != ACT_NONE) v = v * act_derivative<T>(p.act_bwd, side[rr * LDW + c], p.alpha);
                T* c_out = C + i * p.ldc + j;
                if (p.accumulate) v = *c_out + v;
                *c_out = v;
            }
            wave_sync();
        }
        return;
    }

    coordinates();
#pragma unroll
    for (int x = 0; x < WTM; ++x) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int64_t i = row0 + wm * WS + x * 16 + MF::row(r, g);
#pragma unroll
            for (int y = 0; y < WTN; ++y) {
                const int64_t j = col0 + wn * WS + y * 16 + li;
                if (i >= p.M || j >= p.N) continue;
                T v = acc[x][y][r];
                T* c = C + i * p.ldc + j;
                if (p.accumulate) v = *c + v;
                *c = v;
            }
        }
    }
}

template <typename T, int WT, bool A_KC, bool B_KC, bool EDGE, int EPI>
__global__ void __launch_bounds__(GEMM_THREADS, min_blocks(WT)) gemm_kernel(const GemmArgs<T> p, const int tilesM,
                                                                            const int tilesN) {
    GridPos g{blockIdx.x, blockIdx.y, blockIdx.z, gridDim.y, gridDim.z};
    if (WT == 4 && p.shared_splits > 1) {
        // The first workgroups of the launch share the first tiles, shared_splits consecutive workgroups per tile;
        // the rest take one unsplit tile each.
        const unsigned head = (unsigned)p.shared_tiles * (unsigned)p.shared_splits;
        if (blockIdx.x < head) {
            g.bx = blockIdx.x / (unsigned)p.shared_splits;
            g.bz = blockIdx.x % (unsigned)p.shared_splits;
            g.gz = (unsigned)p.shared_splits;
        } else {
            g.bx = (unsigned)p.shared_tiles + (blockIdx.x - head);
        }
    }
    __shared__ __attribute__((aligned(16))) T lds[gemm_lds_elems<T, WT, A_KC, B_KC>()];
    gemm_tile<T, WT, A_KC, B_KC, EDGE, EPI>(p, tilesM, tilesN, g, lds);
}

// 128 x 128 tiles on slabs of half the depth, three workgroups to a compute unit.
template <typename T, bool A_KC, bool B_KC, int EPI>
__global__ void __launch_bounds__(GEMM_THREADS, 3) gemm_thin_kernel(const GemmArgs<T> p, const int tilesM, const int tilesN) {
    __shared__ __attribute__((aligned(16))) T lds[gemm_lds_elems<T, 4, A_KC, B_KC, false, 2>()];
    gemm_tile<T, 4, A_KC, B_KC, false, EPI, false, 2>(p, tilesM, tilesN,
                                                      GridPos{blockIdx.x, blockIdx.y, blockIdx.z, gridDim.y, gridDim.z}, lds);
}

template <typename T, int WT, bool A_KC, bool B_KC>
__global__ void __launch_bounds__(GEMM_THREADS, 4) gemm_short_kernel(const GemmArgs<T> p, const int tilesM, const int tilesN) {
    __shared__ __attribute__((aligned(16))) T lds[gemm_lds_elems<T, WT, A_KC, B_KC, true>()];
    gemm_tile<T, WT, A_KC, B_KC, true, EPI_PLAIN, true>(p, tilesM, tilesN,
                                                        GridPos{blockIdx.x, blockIdx.y, blockIdx.z, gridDim.y, gridDim.z}, lds);
}

// The two gradient products of a layer, dA = dC . B^T (both operands k-contiguous; the upstream activation's
// backward may be its epilogue) and dB = A^T . dC (both operands mn-contiguous; the bias gradient may ride along),
// in one launch on tiles of one size (WT = 1, 2, 4): small layers cost what their chain of dependent launches
// costs, and the launch ramp, first slab and epilogue of one product hide behind the other's main loop.  Workgroups
// [0, first) belong to the first product, the rest to the second.  Neither product is split or batched.
template <typename T, int WT, bool EDGE1, int EPI1, bool EDGE2>
__global__ void __launch_bounds__(GEMM_THREADS, 2) gemm_pair_kernel(const GemmArgs<T> p1, const int tilesM1, const int tilesN1,
                                                                     const GemmArgs<T> p2, const int tilesM2, const int tilesN2,
                                                                     const unsigned first) {
    // (one block of LDS serves whichever product the workgroup belongs to, so two workgroups fit on a compute unit)
    constexpr int LDS1 = gemm_lds_elems<T, WT, true, true>(), LDS2 = gemm_lds_elems<T, WT, false, false>();
    __shared__ __attribute__((aligned(16))) T lds[LDS1 > LDS2 ? LDS1 : LDS2];
    if (blockIdx.x < first) gemm_tile<T, WT, true, true, EDGE1, EPI1>(p1, tilesM1, tilesN1, GridPos{blockIdx.x, 0u, 0u, 1u, 1u}, lds);
    else gemm_tile<T, WT, false, false, EDGE2, EPI_PLAIN>(p2, tilesM2, tilesN2, GridPos{blockIdx.x - first, 0u, 0u, 1u, 1u}, lds);
}

// Which products go to the single-stage kernel (PRAD_GEMM_SHORT=0 switches it off: tuning aid): batches of small
// products whose K fits one slab.  (128 x 128 tiles of three K slabs, a thousand of them, were measured on it too,
// three workgroups to a compute unit: 10 to 25 % slower than the pipelined kernel at two.)
template <typename T, int WT>
static bool gemm_short_eligible(const GemmArgs<T>& a, int epi) {
    static const bool enabled = [] { const char* e = getenv("PRAD_GEMM_SHORT"); return !(e && e[0] == '0'); }();
    return enabled && WT != 4 && epi == EPI_PLAIN && a.ksplit == 0 && a.colsum_dst == nullptr && a.K <= Slab<T, WT>::BK &&
           a.batch >= 64;
}

// Products of very few K slabs on hundreds of 128 x 128 tiles (a layer of 96 inputs applied to tens of thousands of
// rows) go to the half-depth kernel in float: measured on such layers 4 to 25 % faster per launch (most with an
// elementwise epilogue), while K = 256 on a thousand tiles is 5 % slower on it, and in double, where a slab is
// half as deep to begin with, the same layers are 15 to 25 % slower on it.  PRAD_GEMM_THIN_MAX_K overrides the largest K that goes there (0 switches the
// kernel off), PRAD_GEMM_THIN_MIN_TILES the smallest tile count: tuning aids.
template <typename T>
static bool gemm_thin_eligible(const GemmArgs<T>& a, bool edge, int epi, int64_t tiles) {
    static const int64_t max_k = [] { const char* e = getenv("PRAD_GEMM_THIN_MAX_K"); return e ? (int64_t)atoll(e) : (int64_t)128; }();
    static const int64_t min_tiles = [] { const char* e = getenv("PRAD_GEMM_THIN_MIN_TILES"); return e ? (int64_t)atoll(e) : (int64_t)384; }();
    // A K of up to 384 goes there too while the tiles are no more than the full-depth kernel's 512 slots (two
    // workgroups per compute unit): all tiles are resident at once either way, and three half-depth workgroups per
    // compute unit start the later ones' loads sooner (the attention block's 288- and 384-deep layers on 392 tiles: +1 %
    // on the step); on a thousand tiles, two full rounds of the full-depth kernel, K = 256 was measured 5 % slower.
    static const int64_t one_round_max_k = [] { const char* e = getenv("PRAD_GEMM_THIN_ONE_ROUND_MAX_K"); return e ? (int64_t)atoll(e) : (int64_t)384; }();
    const int64_t k_limit = (max_k > 0 && tiles * a.batch <= 512 && one_round_max_k > max_k) ? one_round_max_k : max_k;
    if (edge || a.ksplit != 0 || a.shared_splits > 1 || a.colsum_dst != nullptr || a.K > k_limit || (PRAD_GEMM_FOLD_K > 0 && a.K > PRAD_GEMM_FOLD_K) || tiles * a.batch < min_tiles) return false;  // (no fold on it)
    return epi == EPI_PLAIN || epi == EPI_ELEMENTWISE;
}

template <typename T, int WT, bool A_KC, bool B_KC>
static hipError_t launch_layout(const GemmArgs<T>& a, bool edge, int epi, hipStream_t stream) {
    constexpr int BM = 32 * WT;
    const int tilesM = (int)((a.M + BM - 1) / BM), tilesN = (int)((a.N + BM - 1) / BM);
    const unsigned splits = (a.ksplit > 0 && a.shared_splits <= 1) ? (unsigned)((a.K + a.ksplit - 1) / a.ksplit) : 1u;
    const unsigned riders = a.colsum_dst != nullptr ? (unsigned)((a.colsum_cols + 63) / 64) : 0u;
    dim3 grid((unsigned)(tilesM * tilesN) + riders, (unsigned)a.batch, splits), block(GEMM_THREADS, 1, 1);
    if (WT == 4 && a.shared_splits > 1) grid.x = (unsigned)(tilesM * tilesN) + (unsigned)a.shared_tiles * (unsigned)(a.shared_splits - 1);
    if constexpr (WT == 4 && sizeof(T) == 4) {
        if (gemm_thin_eligible<T>(a, edge, epi, (int64_t)tilesM * tilesN)) {
            if (epi == EPI_PLAIN) hipLaunchKernelGGL((gemm_thin_kernel<T, A_KC, B_KC, EPI_PLAIN>), grid, block, 0, stream, a, tilesM, tilesN);
            else hipLaunchKernelGGL((gemm_thin_kernel<T, A_KC, B_KC, EPI_ELEMENTWISE>), grid, block, 0, stream, a, tilesM, tilesN);
            return hipGetLastError();
        }
    }
    if constexpr (WT != 4) {
        if (gemm_short_eligible<T, WT>(a, epi)) {
            hipLaunchKernelGGL((gemm_short_kernel<T, WT, A_KC, B_KC>), grid, block, 0, stream, a, tilesM, tilesN);
            return hipGetLastError();
        }
    }
#define PRAD_LAUNCH(EDGE_, EPI_) \
    hipLaunchKernelGGL((gemm_kernel<T, WT, A_KC, B_KC, EDGE_, EPI_>), grid, block, 0, stream, a, tilesM, tilesN)
    if (edge) {
        if (epi == EPI_PLAIN) PRAD_LAUNCH(true, EPI_PLAIN);
        else if (epi == EPI_ELEMENTWISE) PRAD_LAUNCH(true, EPI_ELEMENTWISE);
        else PRAD_LAUNCH(true, EPI_TILE_SUM);
    } else {
        if (epi == EPI_PLAIN) PRAD_LAUNCH(false, EPI_PLAIN);
        else if (epi == EPI_ELEMENTWISE) PRAD_LAUNCH(false, EPI_ELEMENTWISE);
        else PRAD_LAUNCH(false, EPI_TILE_SUM);
    }
#undef PRAD_LAUNCH
    return hipGetLastError();
}

// The unguarded kernels use 16-byte loads (any M, N, K: tiles over the edge clamp their loads, a ragged end of K
// is handled inside); they need operands whose rows start 16-byte aligned.  The tile-sum epilogue adds up whole
// tiles and therefore needs the zero fill of the guarded kernels when the output does not fill its tiles.
template <typename T>
static bool vector_loads_ok(const GemmArgs<T>& a, int epi, int BM) {
    constexpr int VEC = Mfma<T>::VEC;
    const bool whole = (a.M % BM == 0) && (a.N % BM == 0);
    return (whole || epi != EPI_TILE_SUM) && a.K > 0 && (a.lda % VEC == 0) &&
           (a.ldb % VEC == 0) && (reinterpret_cast<uintptr_t>(a.A) % 16 == 0) &&
           (reinterpret_cast<uintptr_t>(a.B) % 16 == 0) && (a.strideA % VEC == 0) && (a.strideB % VEC == 0) &&
           (a.zstrideA % VEC == 0) && (a.zstrideB % VEC == 0) && (a.istrideA % VEC == 0) && (a.istrideB % VEC == 0) &&
           // per-thread byte offsets inside one tile's slab are kept in 32 bits
           (a.lda < (1 << 21)) && (a.ldb < (1 << 21));
}

template <typename T, int WT>
static hipError_t launch_tile(const GemmArgs<T>& a, int epi, hipStream_t stream) {
    constexpr int BM = 32 * WT;
    const bool aligned = vector_loads_ok(a, epi, BM);
    // Grid y carries the batch; the tile count must fit the 1-D grid.
    if ((int64_t)((a.M + BM - 1) / BM) * ((a.N + BM - 1) / BM) > 0x7fffffffLL || a.batch > 65535) return hipErrorInvalidValue;
    if (!a.transA && !a.transB) return launch_layout<T, WT, true, false>(a, !aligned, epi, stream);
    if (!a.transA && a.transB) return launch_layout<T, WT, true, true>(a, !aligned, epi, stream);
    return launch_layout<T, WT, false, false>(a, !aligned, epi, stream);
}

enum TileShape { TILE_128x128, TILE_64x64, TILE_32x32 };

// Output tile for a product: the largest tile that still yields one workgroup per compute unit, so
// that small products are spread over the whole chip (measured in double: N = 1024 runs 2.6x faster
// on 64 x 64 tiles than on 128 x 128, N = 512 4.8x faster on 32 x 32; a 128 x 64 tile was measured at
// N = 2048 and 4096 and was never faster than 128 x 128).  PRAD_GEMM_TILE=128x128|64x64|32x32 in the
// environment overrides the choice (a tuning aid).
static TileShape choose_tile(int64_t M, int64_t N, int64_t K, int batch, bool tile_sums, int elem_size) {
    if (tile_sums) return TILE_128x128;  // the tile_sums layout is defined on 128 x 128 tiles
    static const int forced = []() {
        const char* e = getenv("PRAD_GEMM_TILE");
        if (!e) return -1;
        if (!strcmp(e, "128x128")) return (int)TILE_128x128;
        if (!strcmp(e, "64x64")) return (int)TILE_64x64;
        if (!strcmp(e, "32x32")) return (int)TILE_32x32;
        return -1;
    }();
    if (forced >= 0) return (TileShape)forced;
    // Work actually multiplied when the output is padded to whole tiles of edge e.
    auto padded = [&](int64_t e) { return ((M + e - 1) / e * e) * ((N + e - 1) / e * e); };
    auto tiles = [&](int64_t e) { return ((M + e - 1) / e) * ((N + e - 1) / e) * batch; };
    const int64_t least = padded(32) < padded(64) ? (padded(32) < padded(128) ? padded(32) : padded(128))
                                                  : (padded(64) < padded(128) ? padded(64) : padded(128));
    // A tile is admissible unless padding makes it multiply more than twice the best choice's work (a 49 x 49
    // product must not run on a 128 x 128 tile, but a 96-wide output is still faster on it: measured);
    // among the admissible ones take the largest that still gives 256 workgroups - the 64 x 64 tile already from 192
    // (double) or 144 (float) workgroups: forward and backward of square products, 64 x 64 against 32 x 32 tiles, ran
    // +46 % / +12 % (float / double) at N = 960 (225 tiles), +25 / +8 % at 896 (196), +29 / -4 % at 832 (169), +7 / -13 %
    // at 768 (144), -6 / -10 % at 640 (100); the 128 x 128 tile against the 64 x 64 one is level at N = 1920 (225 tiles)
    // and 6 to 8 % behind at 1792 (196), so its threshold stays.
    auto ok = [&](int64_t e) { return padded(e) <= 2 * least; };
    // Past 256 tiles of 128 x 128 the launch is rounds of unequal fill: 400 tiles put two workgroups on some compute
    // units and one on the rest and last as long as 512; 784 tiles last as long as 1024.  Forward and backward at
    // N = 2304 (324 tiles) ran at 61 % of peak in double, at 2560 (400) at 75 %, at 3584 (784) at 73 %, at 3840 (900) at
    // 85 %, while four times as many 64 x 64 tiles, spread more evenly, reach 84, 89, 91 and 90 % (float: 70, 72, 72
    // and 82 % against 77, 83, 87 and 86 %).  Where the large tile fills its rounds it stays ahead: N = 2816 (484
    // tiles) 90 against 84 %, 3328 (676, the last 164 shared three ways, see gemm_shared_tiles_plan) 93 against 91 %,
    // 4096 96.3 against 95.4 %, 5120 95 against 84 %.  The model that reproduces every one of these: a compute unit works through its
    // workgroups at one rate however many it holds, so t tiles last ceil(t / 256) rounds (a shared last round:
    // ceil(rest * ways / 256) / ways), and the tile with the better work / rounds times its own efficiency wins
    // (0.956, shared 0.94, against 0.90 in double; 0.93, 0.885 against 0.87 in float: the small tile's own figure was
    // measured between 0.84 and 0.95 from one machine and size to the next - it moves twice the bytes per flop and
    // falls to 0.83 at N = 6144 - so it is set where the clear cases above go its way and the close ones do not).
    // Only for a K of a thousand or more: shallow products on hundreds of tiles have the half-depth kernel,
    // measured on the large tile.
    if (ok(128) && ok(64) && K >= 1024 && tiles(128) > 256) {
        const int64_t t = tiles(128), q = t / 512, rest = t % 512;
        double rounds = (double)((t + 255) / 256);
        bool shared = false;
        if (t >= 512 && rest != 0 && rest <= 256 && batch == 1) {
            const int64_t bk = elem_size == 8 ? Slab<double, 4>::BK : Slab<float, 4>::BK;
            int64_t ways = 512 / rest < 4 ? 512 / rest : 4;
            if (ways > K / (8 * bk)) ways = K / (8 * bk);
            if (ways >= 2) {
                shared = true;
                rounds = 2.0 * (double)q + (double)((rest * ways + 255) / 256) / (double)ways;
            }
        }
        const bool f32 = elem_size == 4;
        const double large = (double)t / 256.0 / rounds * (shared ? (f32 ? 0.885 : 0.94) : (f32 ? 0.93 : 0.956));
        const int64_t t64 = tiles(64);
        const double small = (double)t64 / (double)((t64 + 255) / 256 * 256) * (f32 ? 0.87 : 0.90);
        return small > large ? TILE_64x64 : TILE_128x128;
    }
    if (ok(128) && tiles(128) >= 256) return TILE_128x128;
    if (ok(64) && tiles(64) >= (elem_size == 4 ? 144 : 192)) return TILE_64x64;
    if (ok(32)) return TILE_32x32;
    return ok(64) ? TILE_64x64 : TILE_128x128;
}

// Splitting K buys parallelism for products with few output tiles, at the price of a second launch
// (the reduce) and a round trip of the partial results through memory: it pays only when the
// unsplit K loop is long.  PRAD_GEMM_SPLIT_MIN_SLABS overrides the threshold (tuning aid).
static int split_min_slabs() {
    static const int v = [] {
        const char* e = getenv("PRAD_GEMM_SPLIT_MIN_SLABS");
        const int x = e ? atoi(e) : 0;
        return x > 0 ? x : 6;
    }();
    return v;
}

int gemm_split_factor(int64_t M, int64_t N, int64_t K, int batch, int elem_size) {
    const int64_t tiles = ((M + 31) / 32) * ((N + 31) / 32) * batch;  // the smallest tile is what such products get
    if (tiles >= 192) return 1;
    const int64_t bk = (elem_size == 8 ? Slab<double, 1>::BK : Slab<float, 1>::BK);
    if ((K + bk - 1) / bk < split_min_slabs()) return 1;
    static const int max_splits = [] { const char* e = getenv("PRAD_GEMM_SPLIT_MAX"); const int x = e ? atoi(e) : 0; return x > 0 ? x : 32; }();
    int64_t s = 512 / tiles;
    if (s > max_splits) s = max_splits;
    if (s > K / (2 * bk)) s = K / (2 * bk);  // at least two slabs per split
    if (s < 2) return 1;
    const int64_t ksplit = ((K + s - 1) / s + bk - 1) / bk * bk;
    return (int)((K + ksplit - 1) / ksplit);
}

static int64_t slab_depth(TileShape t, int elem_size) {
    if (elem_size == 8) return t == TILE_128x128 ? Slab<double, 4>::BK : t == TILE_64x64 ? Slab<double, 2>::BK : Slab<double, 1>::BK;
    return t == TILE_128x128 ? Slab<float, 4>::BK : t == TILE_64x64 ? Slab<float, 2>::BK : Slab<float, 1>::BK;
}

// A product whose chosen tile yields between half and one and a half workgroups per compute unit leaves
// workgroup slots empty (two fit per compute unit).  Such a product on the 64 x 64 or 32 x 32 tile, with a K of 32
// slabs or more, can run as pairs of workgroups per tile, half of K each.  That paid (+4 to +20 %) as long as a lone
// workgroup left the matrix core idle while it moved its slabs; since the main loop issues those transfers between its
// MFMAs a lone workgroup is the faster one everywhere it was measured (N = 1024 in double: 40 us against 45 us paired;
// 1536 x 1024 x 1024: 67 against 70), so pairing is off unless PRAD_GEMM_PAIRS=1 asks for it (a tuning aid; the
// exchange is the one of the products split along K).  The 128 x 128 tile never pairs.
bool gemm_pairs(int64_t M, int64_t N, int64_t K, int batch, int elem_size) {
    static const bool enabled = [] { const char* e = getenv("PRAD_GEMM_PAIRS"); return e && e[0] == '1'; }();
    if (!enabled || gemm_split_factor(M, N, K, batch, elem_size) > 1) return false;
    const TileShape t = choose_tile(M, N, K, batch, false, elem_size);
    const int64_t e = t == TILE_128x128 ? 128 : t == TILE_64x64 ? 64 : 32;
    const int64_t wgs = ((M + e - 1) / e) * ((N + e - 1) / e) * batch;
    return t != TILE_128x128 && wgs >= 128 && wgs <= GEMM_SPLIT_MAX_TILES && K >= 32 * slab_depth(t, elem_size);
}

// A product of few 128 x 128 tiles and a long K (a weight gradient over thousands of rows: 256 x 2048 with K = 8192
// is 32 such tiles) would run on 64 x 64 or 32 x 32 tiles to fill the chip, at their lower ratio of MFMAs to LDS
// traffic.  With K long enough every 128 x 128 tile is shared by `ways` workgroups instead (the mechanism of
// gemm_shared_tiles_plan with all tiles shared): four ways or more, at least 192 workgroups, at least 32 slabs of K
// each, little padding.
// Returns the ways (0: not such a product) and the number of tiles.
static int few_tiles_long_k_plan(int64_t M, int64_t N, int64_t K, int elem_size, int* tiles_out) {
    static const bool enabled = [] { const char* e = getenv("PRAD_GEMM_FEW_TILES"); return !(e && e[0] == '0'); }();  // tuning aid
    if (!enabled || choose_tile(M, N, K, 1, false, elem_size) == TILE_128x128) return 0;
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    if (tiles * 128 * 128 * 4 > M * N * 5) return 0;  // more than a quarter of padding: the smaller tiles multiply less
    const int64_t bk = slab_depth(TILE_128x128, elem_size);
    int64_t ways = 256 / tiles;
    if (ways > 16) ways = 16;
    if (ways > K / (32 * bk)) ways = K / (32 * bk);
    // (two ways were measured level with the smaller tiles once the launch that adds the partial tiles is counted:
    // 8192 x 256 with K = 2048, 70.9 + 7.4 us against 69.5)
    if (ways < 4 || tiles * ways < 192) return 0;
    *tiles_out = (int)tiles;
    return (int)ways;
}

int gemm_shared_tiles_plan(int64_t M, int64_t N, int64_t K, int batch, int elem_size, int* shared_tiles) {
    static const bool enabled = [] { const char* e = getenv("PRAD_GEMM_SHARED"); return !(e && e[0] == '0'); }();  // tuning aid
    *shared_tiles = 0;
    if (!enabled || batch != 1) return 0;
    if (gemm_split_factor(M, N, K, batch, elem_size) > 1) return 0;
    if (const int ways = few_tiles_long_k_plan(M, N, K, elem_size, shared_tiles)) return ways;
    if (choose_tile(M, N, K, batch, false, elem_size) != TILE_128x128) return 0;
    constexpr int64_t SLOTS = 512;  // two workgroups of the 128 x 128 kernels per compute unit
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    // (fewer tiles than slots - 256 tiles, one per compute unit - were measured with every tile shared two ways: +2 %,
    // the partial tiles' round trip eats what the second workgroup per compute unit gains; not done)
    const int64_t rest = tiles % SLOTS;
    if (tiles < SLOTS || rest == 0 || rest > SLOTS / 2) return 0;  // a last round that is at least half full is left alone
    const int64_t bk = slab_depth(TILE_128x128, elem_size);
    static const int64_t max_ways = [] { const char* e = getenv("PRAD_GEMM_SHARED_MAX_WAYS"); const int x = e ? atoi(e) : 0; return (int64_t)(x > 1 ? x : 4); }();
    int64_t ways = SLOTS / rest;
    if (ways > max_ways) ways = max_ways;
    if (ways > K / (8 * bk)) ways = K / (8 * bk);  // at least eight slabs per workgroup
    if (ways < 2) return 0;
    *shared_tiles = (int)rest;
    return (int)ways;
}

// Adds the partial results of a split product in split order and applies the epilogue.
template <typename T>
__global__ void __launch_bounds__(256) split_reduce_kernel(const GemmArgs<T> p, const T* __restrict__ ws, int splits) {
    const int64_t mn = p.M * p.N, total = mn * p.batch;
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int64_t b = idx / mn, e = idx % mn, i = e / p.N, j = e % p.N;
        T v = ws[idx];
        for (int z = 1; z < splits; ++z) v = v + ws[(int64_t)z * total + idx];
        if (p.bias != nullptr) v = v + p.bias[j];
        if (p.Z != nullptr) p.Z[i * p.ldz + j] = v;
        if (p.act_fwd != ACT_NONE) v = act_forward<T>(p.act_fwd, v, p.alpha);
        if (p.act_bwd != ACT_NONE) v = v * act_derivative<T>(p.act_bwd, p.act_src[i * p.ld_act + j], p.alpha);
        T* c = p.C + b * p.strideC + i * p.ldc + j;
        if (p.accumulate) v = *c + v;
        *c = v;
    }
}

// Adds the partial blocks of the shared tiles of a launch (see gemm_shared_tiles_plan) in split order and applies the
// epilogue.  One workgroup takes 16 rows of one tile, a thread one 16-byte vector of eight rows of them.
template <typename T>
__global__ void __launch_bounds__(256) shared_reduce_kernel(const GemmArgs<T> p, const int tilesM, const int tilesN) {
    typedef typename Mfma<T>::Vec Vec;
    constexpr int VEC = Mfma<T>::VEC, BM = 128, BN = 128, VPR = BN / VEC;  // vectors per tile row
    const int tile = blockIdx.x / (BM / 16), strip = blockIdx.x % (BM / 16);
    int tm, tn;
    tile_of_workgroup(tile, tilesM, tilesN, tm, tn);
    const int64_t row0 = (int64_t)tm * BM, col0 = (int64_t)tn * BN;
    const int splits = p.shared_splits;
    const T* __restrict__ ws = p.split_ws + (int64_t)tile * splits * (BM * BN);
    for (int e = threadIdx.x; e < 16 * VPR; e += 256) {
        const int il = strip * 16 + e / VPR, jl = (e % VPR) * VEC;
        const int64_t i = row0 + il, j = col0 + jl;
        if (i >= p.M || j >= p.N) continue;
        Vec v = *reinterpret_cast<const Vec*>(ws + il * BN + jl);
        for (int z = 1; z < splits; ++z) {
            const Vec o = *reinterpret_cast<const Vec*>(ws + (int64_t)z * (BM * BN) + il * BN + jl);
#pragma unroll
            for (int c = 0; c < VEC; ++c) v[c] = v[c] + o[c];
        }
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
            if (j + c >= p.N) break;
            T x = v[c];
            if (p.bias != nullptr) x = x + p.bias[j + c];
            if (p.Z != nullptr) p.Z[i * p.ldz + j + c] = x;
            if (p.act_fwd != ACT_NONE) x = act_forward<T>(p.act_fwd, x, p.alpha);
            if (p.act_bwd != ACT_NONE) x = x * act_derivative<T>(p.act_bwd, p.act_src[i * p.ld_act + j + c], p.alpha);
            T* out = p.C + i * p.ldc + j + c;
            if (p.accumulate) x = *out + x;
            *out = x;
        }
    }
}

template <typename T>
hipError_t launch_gemm(const GemmArgs<T>& a_in, hipStream_t stream) {
    if (a_in.M <= 0 || a_in.N <= 0 || a_in.batch <= 0) return hipSuccess;
    if (a_in.transA && a_in.transB) return hipErrorInvalidValue;
    GemmArgs<T> a = a_in;
    a.ksplit = 0; a.zstrideA = 0; a.zstrideB = 0;
    const int epi = a.tile_sums != nullptr ? EPI_TILE_SUM
                    : (a.bias != nullptr || a.Z != nullptr || a.act_fwd != ACT_NONE || a.act_bwd != ACT_NONE) ? EPI_ELEMENTWISE
                                                                                                             : EPI_PLAIN;
    if constexpr (sizeof(T) == 4) {
        if (epi == EPI_PLAIN) {
            const hipError_t e = launch_gemm_skinny(a, stream);
            if (e != hipErrorNotSupported) return e;
        }
        if (epi != EPI_TILE_SUM) {
            const hipError_t e = launch_gemm_tall(a, stream);
            if (e != hipErrorNotSupported) return e;
        }
    }
    if (a.nseg > 1) {
        // Sum of nseg products: one operand pair per split, partial results added in pair order.
        if (a.split_ws == nullptr || a.batch != 1 || epi == EPI_TILE_SUM) return hipErrorInvalidValue;
        GemmArgs<T> part = a;
        part.split_counters = nullptr;
        part.K = a.K * a.nseg;
        part.ksplit = a.K;
        part.zstrideA = a.segstrideA; part.zstrideB = a.segstrideB;
        part.C = a.split_ws; part.ldc = a.N; part.strideC = a.M * a.N;
        part.accumulate = 0;
        part.bias = nullptr; part.Z = nullptr; part.act_fwd = ACT_NONE; part.act_bwd = ACT_NONE; part.act_src = nullptr;
        hipError_t e;
        switch (choose_tile(a.M, a.N, a.K, a.nseg, false, (int)sizeof(T))) {
            case TILE_128x128: e = launch_tile<T, 4>(part, EPI_PLAIN, stream); break;
            case TILE_64x64: e = launch_tile<T, 2>(part, EPI_PLAIN, stream); break;
            default: e = launch_tile<T, 1>(part, EPI_PLAIN, stream); break;
        }
        if (e != hipSuccess) return e;
        const int64_t total = a.M * a.N;
        int64_t blocks = (total + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL((split_reduce_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream, a, a.split_ws, a.nseg);
        return hipGetLastError();
    }
    int splits = (a.split_ws != nullptr && epi != EPI_TILE_SUM) ? gemm_split_factor(a.M, a.N, a.K, a.batch, (int)sizeof(T)) : 1;
    {
        // the two-pass reduction addresses C with one batch stride
        const int64_t tiles = ((a.M + 31) / 32) * ((a.N + 31) / 32) * a.batch;
        if (a.batch_inner > 1 && !(a.split_counters != nullptr && tiles <= GEMM_SPLIT_MAX_TILES)) splits = 1;
    }
    if (splits > 1) {
        constexpr int64_t bk = Slab<T, 1>::BK;
        const int64_t tiles = ((a.M + 31) / 32) * ((a.N + 31) / 32) * a.batch;
        GemmArgs<T> part = a;
        part.ksplit = ((a.K + splits - 1) / splits + bk - 1) / bk * bk;
        part.zstrideA = a.transA ? part.ksplit * a.lda : part.ksplit;  // A stored [k][m] when transposed, else [m][k]
        part.zstrideB = a.transB ? part.ksplit : part.ksplit * a.ldb;  // B stored [n][k] when transposed, else [k][n]
        if (a.split_counters != nullptr && tiles <= GEMM_SPLIT_MAX_TILES)
            return launch_tile<T, 1>(part, epi, stream);  // one launch: the last workgroup of a tile reduces
        // two passes: partial products, then a kernel that adds them in split order and applies the epilogue
        part.split_counters = nullptr;
        part.C = a.split_ws; part.ldc = a.N; part.strideC = a.M * a.N;  // split z, batch b at ((z * batch) + b) * M * N
        part.accumulate = 0;
        part.bias = nullptr; part.Z = nullptr; part.act_fwd = ACT_NONE; part.act_bwd = ACT_NONE; part.act_src = nullptr;
        hipError_t e = launch_tile<T, 1>(part, EPI_PLAIN, stream);
        if (e != hipSuccess) return e;
        const int64_t total = a.M * a.N * a.batch;
        int64_t blocks = (total + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL((split_reduce_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream, a, a.split_ws, splits);
        return hipGetLastError();
    }
    TileShape tile = choose_tile(a.M, a.N, a.K, a.batch, a.tile_sums != nullptr, (int)sizeof(T));
    a.shared_tiles = 0; a.shared_splits = 0;
    int shared_tiles = 0;
    const int shared_ways = (a.tile_sums == nullptr && a.split_ws != nullptr && epi != EPI_TILE_SUM &&
                             a.batch_inner <= 1 && a.colsum_dst == nullptr)
                                ? gemm_shared_tiles_plan(a.M, a.N, a.K, a.batch, (int)sizeof(T), &shared_tiles) : 0;
    if (shared_ways > 1) {
        tile = TILE_128x128;  // (few tiles and a long K: the plan puts a product of smaller tiles on shared 128 x 128 ones)
        const int64_t bk = slab_depth(tile, (int)sizeof(T));
        a.ksplit = ((a.K + shared_ways - 1) / shared_ways + bk - 1) / bk * bk;
        a.shared_splits = (int)((a.K + a.ksplit - 1) / a.ksplit);
        a.shared_tiles = shared_tiles;
        a.zstrideA = a.transA ? a.ksplit * a.lda : a.ksplit;
        a.zstrideB = a.transB ? a.ksplit : a.ksplit * a.ldb;
        a.split_counters = nullptr;  // the shared tiles are reduced by a launch of their own
        if (a.shared_splits < 2) { a.shared_splits = 0; a.shared_tiles = 0; a.ksplit = 0; }
    } else if (a.split_counters != nullptr && a.split_ws != nullptr && epi != EPI_TILE_SUM &&
        gemm_pairs(a.M, a.N, a.K, a.batch, (int)sizeof(T))) {
        const int64_t bk = slab_depth(tile, (int)sizeof(T));
        a.ksplit = ((a.K + 1) / 2 + bk - 1) / bk * bk;
        a.zstrideA = a.transA ? a.ksplit * a.lda : a.ksplit;
        a.zstrideB = a.transB ? a.ksplit : a.ksplit * a.ldb;
    } else {
        a.split_counters = nullptr;
    }
    switch (tile) {
        case TILE_128x128: {
            const hipError_t e = launch_tile<T, 4>(a, epi, stream);
            if (e != hipSuccess || a.shared_splits <= 1) return e;
            hipLaunchKernelGGL((shared_reduce_kernel<T>), dim3((unsigned)a.shared_tiles * 8u), dim3(256), 0, stream, a,
                               (int)((a.M + 127) / 128), (int)((a.N + 127) / 128));
            return hipGetLastError();
        }
        case TILE_64x64: return launch_tile<T, 2>(a, epi, stream);
        default: return launch_tile<T, 1>(a, epi, stream);
    }
}

// Both gradient products of a layer in one launch (gemm_pair_kernel).  Taken only where each product alone would
// run unsplit on the same tile, so that the results are those of the two separate launches bit for bit.  Measured against the separate launches, forward and backward of square products in float / double:
// N = 768 +21 / +15 %, 1024 +9 / +3 %, 1536 +13 / +12 %, 1792 +9 / +9 % (the tail of one product overlaps the other's
// start; PRAD_GEMM_DUAL_MAX caps the workgroups of such a launch, PRAD_GEMM_DUAL_64=0 keeps the 64 x 64 and 128 x 128 tiles out: tuning
// aids).  hipErrorNotSupported otherwise: the caller then launches the products one after the other.
template <typename T>
hipError_t launch_gemm_pair(const GemmArgs<T>& first_in, const GemmArgs<T>& second_in, hipStream_t stream) {
    static const bool enabled = [] { const char* e = getenv("PRAD_GEMM_DUAL"); return !(e && e[0] == '0'); }();  // tuning aid
    static const bool wide = [] { const char* e = getenv("PRAD_GEMM_DUAL_64"); return !(e && e[0] == '0'); }();  // tuning aid
    if (!enabled) return hipErrorNotSupported;
    GemmArgs<T> p1 = first_in, p2 = second_in;
    auto epilogue = [](const GemmArgs<T>& a) {
        return (a.bias != nullptr || a.Z != nullptr || a.act_fwd != ACT_NONE || a.act_bwd != ACT_NONE) ? EPI_ELEMENTWISE : EPI_PLAIN;
    };
    // (a product that launch_gemm would move to shared 128 x 128 tiles adds its partial tiles in another order)
    auto shared_ways = [](const GemmArgs<T>& a) { int tiles = 0; return gemm_shared_tiles_plan(a.M, a.N, a.K, 1, (int)sizeof(T), &tiles); };
    // (nor one that has a kernel of its own: the streaming kernel for tall products, the one-pass weight gradient)
    auto special = [](const GemmArgs<T>& a) {
        if constexpr (sizeof(T) == 4) return gemm_tall_eligible(a) || gemm_skinny_eligible(a);
        else return false;
    };
    auto small = [shared_ways, special](const GemmArgs<T>& a, TileShape tile) {
        return !special(a) && a.M > 0 && a.N > 0 && a.K > 0 && a.batch == 1 && a.batch_inner <= 1 && a.nseg <= 1 && a.tile_sums == nullptr &&
               choose_tile(a.M, a.N, a.K, 1, false, (int)sizeof(T)) == tile && gemm_split_factor(a.M, a.N, a.K, 1, (int)sizeof(T)) == 1 &&
               !gemm_pairs(a.M, a.N, a.K, 1, (int)sizeof(T)) && shared_ways(a) <= 1;
    };
    if (p1.transA || !p1.transB || !p2.transA || p2.transB || p1.M <= 0 || p1.N <= 0) return hipErrorNotSupported;
    const TileShape tile = choose_tile(p1.M, p1.N, p1.K, 1, false, (int)sizeof(T));
    if ((tile != TILE_32x32 && !wide) || !small(p1, tile) || !small(p2, tile)) return hipErrorNotSupported;
    // (float products of few K slabs on 128 x 128 tiles have the half-depth kernel)
    if (tile == TILE_128x128 && sizeof(T) == 4 && (p1.K <= 384 || p2.K <= 384)) return hipErrorNotSupported;
    if (epilogue(p2) != EPI_PLAIN || p1.colsum_dst != nullptr) return hipErrorNotSupported;
    for (GemmArgs<T>* p : {&p1, &p2}) { p->ksplit = 0; p->zstrideA = 0; p->zstrideB = 0; p->split_counters = nullptr; p->shared_splits = 0; p->shared_tiles = 0; }
    const int edge = tile == TILE_128x128 ? 128 : tile == TILE_64x64 ? 64 : 32;
    const int tilesM1 = (int)((p1.M + edge - 1) / edge), tilesN1 = (int)((p1.N + edge - 1) / edge);
    const int tilesM2 = (int)((p2.M + edge - 1) / edge), tilesN2 = (int)((p2.N + edge - 1) / edge);
    const unsigned first = (unsigned)(tilesM1 * tilesN1);
    const unsigned riders = p2.colsum_dst != nullptr ? (unsigned)((p2.colsum_cols + 63) / 64) : 0u;
    const unsigned total = first + (unsigned)(tilesM2 * tilesN2) + riders;
    static const unsigned max_total = [] { const char* e = getenv("PRAD_GEMM_DUAL_MAX"); const int x = e ? atoi(e) : 0; return x > 0 ? (unsigned)x : ~0u; }();  // tuning aid
    // (on 128 x 128 tiles a product of 512 tiles or more fills both workgroup slots of every compute unit by itself:
    // N = 2048, 256 + 256 tiles, +4 % in float and +1.5 % in double for forward and backward together; N = 2304, 324 + 324, +20 %;
    // N = 2560, 400 + 400, +1 %; N = 3072 and 4096 level within 0.8 %, and left as the launches they were)
    static const unsigned max_total_128 = [] { const char* e = getenv("PRAD_GEMM_DUAL_MAX_128"); const int x = e ? atoi(e) : 0; return x > 0 ? (unsigned)x : 1024u; }();  // tuning aid
    if (total > max_total || (tile == TILE_128x128 && total > max_total_128)) return hipErrorNotSupported;
    const int epi1 = epilogue(p1);
    const bool edge1 = !vector_loads_ok(p1, epi1, edge), edge2 = !vector_loads_ok(p2, EPI_PLAIN, edge);
    const dim3 grid(total), block(GEMM_THREADS);
#define PRAD_LAUNCH(WT_, E1_, EPI_, E2_) \
    hipLaunchKernelGGL((gemm_pair_kernel<T, WT_, E1_, EPI_, E2_>), grid, block, 0, stream, p1, tilesM1, tilesN1, p2, tilesM2, tilesN2, first)
    if (tile != TILE_32x32) {
        // (misaligned operands on these tiles take the separate launches)
        if (edge1 || edge2) return hipErrorNotSupported;
        if (tile == TILE_128x128) {
            if (epi1 == EPI_PLAIN) PRAD_LAUNCH(4, false, EPI_PLAIN, false);
            else PRAD_LAUNCH(4, false, EPI_ELEMENTWISE, false);
        } else {
            if (epi1 == EPI_PLAIN) PRAD_LAUNCH(2, false, EPI_PLAIN, false);
            else PRAD_LAUNCH(2, false, EPI_ELEMENTWISE, false);
        }
    } else if (edge1 || edge2) {
        // misaligned operands: both products on the guarded loads
        if (epi1 == EPI_PLAIN) PRAD_LAUNCH(1, true, EPI_PLAIN, true);
        else PRAD_LAUNCH(1, true, EPI_ELEMENTWISE, true);
    } else {
        if (epi1 == EPI_PLAIN) PRAD_LAUNCH(1, false, EPI_PLAIN, false);
        else PRAD_LAUNCH(1, false, EPI_ELEMENTWISE, false);
    }
#undef PRAD_LAUNCH
    return hipGetLastError();
}

template <typename T>
static bool lstm_operands_aligned(const GemmArgs<T>& a) {
    constexpr int VEC = Mfma<T>::VEC;
    return a.lda % VEC == 0 && a.ldb % VEC == 0 && reinterpret_cast<uintptr_t>(a.A) % 16 == 0 &&
           reinterpret_cast<uintptr_t>(a.B) % 16 == 0 && a.lda < (1 << 21) && a.ldb < (1 << 21) && a.batch == 1;
}

template <typename T>
hipError_t launch_lstm_step_fwd(const GemmArgs<T>& a_in, hipStream_t stream) {
    GemmArgs<T> a = a_in;
    const int64_t H = a.lstm_hidden;
    constexpr int64_t bk = Slab<T, 1>::BK;
    // M x 4H = (M x H) . (H x 4H); whole slabs of K (the gather has no guarded tail) and whole groups of 8 units
    if (a.M <= 0 || H <= 0) return hipSuccess;
    if (a.transA || a.transB || a.K != H || a.N != 4 * H || H % bk != 0 || H % 8 != 0 || !lstm_operands_aligned(a) ||
        (a.M + 31) / 32 * (H / 8) > 0x7fffffffLL)
        return hipErrorNotSupported;
    a.ksplit = 0; a.zstrideA = 0; a.zstrideB = 0; a.split_counters = nullptr; a.colsum_dst = nullptr; a.nseg = 0;
    const int tilesM = (int)((a.M + 31) / 32), tilesN = (int)(H / 8);
    hipLaunchKernelGGL((gemm_kernel<T, 1, true, false, false, EPI_LSTM_FWD>), dim3((unsigned)(tilesM * tilesN)), dim3(GEMM_THREADS), 0,
                       stream, a, tilesM, tilesN);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_lstm_step_bwd(const GemmArgs<T>& a_in, hipStream_t stream) {
    GemmArgs<T> a = a_in;
    const int64_t H = a.lstm_hidden;
    if (a.M <= 0 || H <= 0) return hipSuccess;
    if (a.transA || !a.transB || a.N != H || a.K != 4 * H || !lstm_operands_aligned(a)) return hipErrorNotSupported;
    a.ksplit = 0; a.zstrideA = 0; a.zstrideB = 0; a.colsum_dst = nullptr; a.nseg = 0;
    const int tilesM = (int)((a.M + 31) / 32), tilesN = (int)((H + 31) / 32);
    const int splits = (a.split_ws != nullptr && a.split_counters != nullptr && (int64_t)tilesM * tilesN <= GEMM_SPLIT_MAX_TILES)
                           ? gemm_split_factor(a.M, a.N, a.K, 1, (int)sizeof(T)) : 1;
    if (splits > 1) {
        constexpr int64_t bk = Slab<T, 1>::BK;
        a.ksplit = ((a.K + splits - 1) / splits + bk - 1) / bk * bk;
        a.zstrideA = a.ksplit;   // A stored [m][k]
        a.zstrideB = a.ksplit;   // B stored [n][k]
    } else {
        a.split_counters = nullptr;
    }
    const unsigned gz = a.ksplit > 0 ? (unsigned)((a.K + a.ksplit - 1) / a.ksplit) : 1u;
    hipLaunchKernelGGL((gemm_kernel<T, 1, true, true, false, EPI_LSTM_BWD>), dim3((unsigned)(tilesM * tilesN), 1, gz),
                       dim3(GEMM_THREADS), 0, stream, a, tilesM, tilesN);
    return hipGetLastError();
}

template hipError_t launch_lstm_step_fwd<double>(const GemmArgs<double>&, hipStream_t);
template hipError_t launch_lstm_step_fwd<float>(const GemmArgs<float>&, hipStream_t);
template hipError_t launch_lstm_step_bwd<double>(const GemmArgs<double>&, hipStream_t);
template hipError_t launch_lstm_step_bwd<float>(const GemmArgs<float>&, hipStream_t);
template hipError_t launch_gemm_pair<double>(const GemmArgs<double>&, const GemmArgs<double>&, hipStream_t);
template hipError_t launch_gemm_pair<float>(const GemmArgs<float>&, const GemmArgs<float>&, hipStream_t);
template hipError_t launch_gemm<double>(const GemmArgs<double>&, hipStream_t);
template hipError_t launch_gemm<float>(const GemmArgs<float>&, hipStream_t);

}  // namespace prad
