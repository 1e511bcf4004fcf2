// Tall products in float: C[M x N] = A[M x K] . op(B) with tens of thousands of rows and a small right operand
// (K x N floats fit one compute unit's LDS) - a layer of 96 to 384 units applied to every token of a batch, forward
// (MatrixMultiplyOperation.Forward, src/RMAD/MatrixMultiplyOperation.cs:50-80, with the bias add and activation that
// follow it in the graph) and the input gradient of the same layer (dA = dC . B^T, :94-104, with the upstream
// activation's Backward).  On 128 x 128 output tiles such a product is a single round of workgroups that all load, then
// all multiply, then all store: nothing overlaps, and it runs at a quarter of what either the matrix cores or the
// memory could do.  Here the right operand is resident and the rows stream:
//
//   * every workgroup (one per compute unit, sixteen wavefronts) first copies the whole of B into LDS, already cut into
//     MFMA fragments: element (y, j, i, g, n) is B[16 j + 4 i + g][16 y + n], so that a wavefront's 64 lanes (g, n) read 64
//     consecutive floats for one MFMA step (no bank conflicts; 16-byte reads per lane were measured with 60 % of the LDS
//     cycles lost to conflicts);
//   * the work is cut into units of 16 rows by NYW 16-column tiles (NYW = 4, 3 or 2: many small units, so that a compute
//     unit's four matrix cores get shares that differ by little); a workgroup owns a contiguous range of units
//     and each of its wavefronts takes one unit after another from it, alone (no barrier after the fill).  A lane (m, g) of the
//     wavefront loads 16 bytes A[row0 + m][16 j + 4 g .. + 3] straight into registers, 96 columns of a unit at a time, each
//     half of them fetched again (for the next 96 columns, or the next unit) as soon as its MFMAs are issued, so a load has
//     the other half's multiplications to arrive.  Before its MFMAs a vector is transposed across the wavefront's four
//     lane groups (four lane-swap instructions per sixteen k), after which element i of lane group g is
//     A[row0 + m][16 j + 4 i + g]: MFMA step 4 j + i then sees k = 4 (4 j + i) + g, the assignment of the tiled kernels;
//   * the MFMA takes the B fragment as its first operand and the A fragment as its second: the 16 x 16 result is then
//     C^T, and a lane holds C[row0 + m][16 y + 4 g .. + 3] - four neighbours of one row - so bias, pre-activation copy,
//     activation, the upstream activation's derivative and the store are all 16-byte accesses with no trip through LDS.
//
// Per element the arithmetic is that of the tiled kernels' elementwise epilogue, in the same order, and the sum along K is
// the same chain of MFMA steps over the same k (K <= 384 here: the float kernels' folding every 512 does not come into
// it): a product has the same bits whichever kernel its shape selects.
#include "common.h"

#include <cstdlib>


namespace prad {

namespace {

typedef float f4t __attribute__((ext_vector_type(4)));

constexpr int TALL_THREADS = 1024;
constexpr int TALL_WAVES = TALL_THREADS / 64;
constexpr int TALL_CH = 6;                       // 16-wide k groups per chunk: 96 columns of A per load round
constexpr int HALF = TALL_CH / 2;
constexpr size_t TALL_MAX_B = 144 * 1024;        // K * N * 4 bytes at most (96 x 384, 384 x 96)
constexpr size_t TALL_MAX_LDS = TALL_MAX_B + 2048;  // and the bias, N <= 384 floats
constexpr int64_t TALL_MIN_ROWS = 8192;

struct TallArgs {
    const float* A; const float* B; float* C;
    const float* bias; float* Z; const float* act_src;
    long lda, ldb, ldc, ldz, ld_act;
    int M, N, K;
    int transB, accumulate, act_fwd, act_bwd;
    float alpha;
    int blocks;  // 16-row blocks in all
    int parts;   // column parts per block: N / 16 / NYW
};

__device__ __forceinline__ f4t load16(const float* base, unsigned byte_offset) {
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, -1, 0x00020000);
    return __builtin_bit_cast(f4t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)byte_offset, 0, 0));
}

// What follows a unit's multiplications.  TALL_STORE: store (or add into) C, with the bias if there is one: straight-line
// code, a few instructions per 16 bytes.  TALL_GENERAL: everything (pre-activation copy, activation, upstream activation's
// derivative) in a runtime loop, see `finish_general`.
// TALL_GELU_FWD / TALL_GELU_BWD: the general epilogue with the activation known at compile time (GELU forward with or
// without the pre-activation copy; GELU's derivative of a cached operand): no dispatch per element, and the four elements
// of a lane's vector are independent instruction chains that the compiler interleaves.
constexpr int TALL_STORE = 0, TALL_GENERAL = 1, TALL_GELU_FWD = 2, TALL_GELU_BWD = 3;

// NYW: 16-column tiles (accumulators per lane) of a unit.  ONE_CHUNK: K == 96, every pass of the main loop is a whole unit.
template <int NYW, int EPI, bool ONE_CHUNK>
__global__ void __launch_bounds__(TALL_THREADS, 1) gemm_tall_kernel(const TallArgs p) {
    extern __shared__ __attribute__((aligned(16))) float bfrag[];  // [y][j][i][g][n] = B[16 j + 4 i + g][16 y + n], then the bias, then the unit counter
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // (said to be uniform: loop counts and load bases that depend on it stay scalar)
    const int li = lane & 15, g = lane >> 4;
    const int KJ = p.K / 16;

    // ---- units: the workgroup owns [first, first + count); wavefront w starts with unit w and then takes the next unit
    // nobody has taken yet (a counter in LDS), so that all sixteen finish within a unit of each other ----
    const int units = p.blocks * p.parts;
    const int first = (int)((long)blockIdx.x * units / gridDim.x);
    const int count = (int)((long)(blockIdx.x + 1) * units / gridDim.x) - first;
    const int nchunks = KJ / TALL_CH;
    const bool working = wave < count;
    int* next_counter = reinterpret_cast<int*>(bfrag + p.K * p.N + p.N);
    if (tid == 0) *next_counter = TALL_WAVES;  // (published by the barrier after the copy of B)

    // lane part of the A address: row li of the unit's block, 16 bytes at k = 4 g of a 16-wide group
    auto a_offset = [&](int unit) {
        const int row = min(16 * (unit / p.parts) + li, p.M - 1);  // rows past the end repeat the last one; they are never stored
        return (unsigned)(((long)row * p.lda + 4 * g) * 4);
    };
    f4t a[TALL_CH];
    // half a chunk's loads: the registers are refilled as soon as the MFMAs that read them have been issued
    auto load_half = [&](int unit, int c, int h) {
        const unsigned off = a_offset(unit);
#pragma unroll
        for (int j = 0; j < HALF; ++j) a[h * HALF + j] = load16(p.A + (c * TALL_CH + h * HALF + j) * 16, off);
    };

    // (the first unit's rows are on their way while B is copied)
    if (working) {
        load_half(first + wave, 0, 0);
        load_half(first + wave, 0, 1);
    }

    // ---- B -> LDS as fragments.  One 16-byte load per lane and step; a wavefront's 64 lanes take one (y, j) pair, the
    // 256 consecutive floats of the fragment array, so that its LDS stores fall on distinct banks (walking B row by row
    // instead had the 64 lanes of a store 16 deep on the same banks).  Up to nine loads are in flight per thread, which is
    // all of the largest B in one round: the copy is latency, not volume.
    {
        constexpr int FILL = 9;
        static_assert(TALL_MAX_B / 16 <= (size_t)FILL * TALL_THREADS, "one round copies the largest B");
        const int npairs = (p.N / 16) * KJ;  // = K * N / 256
        const int l = lane;
        // the lane's part of a pair's addresses (the pair's part, from the wavefront's number, is scalar arithmetic: every
        // vector instruction here is time the float MFMAs of other wavefronts do not get: the two do not overlap on this chip)
        const long lane_at = p.transB ? (long)(l & 15) * p.ldb + 4 * (l >> 4) : (long)(4 * (l >> 4) + ((l >> 2) & 3)) * p.ldb + 4 * (l & 3);
        const int lane_dst = (l >> 4) * 64 + ((l >> 2) & 3) * 16 + 4 * (l & 3);
        for (int pair0 = wave; pair0 < npairs; pair0 += FILL * TALL_WAVES) {
            f4t x[FILL];
#pragma unroll
            for (int u = 0; u < FILL; ++u) {
                const int pair = min(pair0 + u * TALL_WAVES, npairs - 1), y = pair / KJ, j = pair - y * KJ;
                // transposed B is stored [n][k]: lane (gg, nn) reads the four i of (j, gg) for column 16 y + nn;
                // plain B is stored [k][n]: lane (i, gg, n4) reads four neighbouring columns of row k = 16 j + 4 i + gg
                const long pair_at = p.transB ? (long)(16 * y) * p.ldb + 16 * j : (long)(16 * j) * p.ldb + 16 * y;
                x[u] = *reinterpret_cast<const f4t*>(p.B + pair_at + lane_at);
            }
#pragma unroll
            for (int u = 0; u < FILL; ++u) {
                const int pair = pair0 + u * TALL_WAVES;
                if (pair >= npairs) continue;
                float* dst = bfrag + pair * 256;
                if (p.transB) {
                    // the lane holds k = 16 j + 4 q + i for q = l >> 4, i = 0..3: element i belongs to lane group i of step q.
                    // The four are written in an order rotated by q, so that the lanes of a store fall on distinct banks.
                    const int q = l >> 4, n = l & 15;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int e = (i + q) & 3;
                        const float v = e == 0 ? x[u][0] : e == 1 ? x[u][1] : e == 2 ? x[u][2] : x[u][3];
                        dst[q * 64 + e * 16 + n] = v;
                    }
                } else {
                    *reinterpret_cast<f4t*>(dst + lane_dst) = x[u];
                }
            }
        }
    }
    if (p.bias != nullptr)
        for (int n = tid; n < p.N; n += TALL_THREADS) bfrag[p.K * p.N + n] = p.bias[n];
    __syncthreads();

    if (!working) return;
    f4t acc[NYW];
    // A lane (m, g) loaded A[m][16 j + 4 g + e], e = 0..3, in one vector; MFMA step q of the group needs A[m][16 j + 4 q + g]
    // in lane group g (the assignment of k to steps and lane groups that the tiled kernels use: k = 4 s + g, s ascending).
    // That is a 4 x 4 transpose between the vector's elements and the wavefront's four lane groups: two swaps of lane
    // halves, then two swaps of odd with even groups, four instructions per sixteen k.
    auto transpose_k = [](f4t& v) {
        typedef unsigned u2t __attribute__((ext_vector_type(2)));
        // (element by element through plain floats: a bit cast applied to a vector element reads element 0)
        const float f0 = v[0], f1 = v[1], f2 = v[2], f3 = v[3];
        unsigned r0 = __float_as_uint(f0), r1 = __float_as_uint(f1), r2 = __float_as_uint(f2), r3 = __float_as_uint(f3);
        u2t t;
        t = __builtin_amdgcn_permlane32_swap(r0, r2, false, false); r0 = t[0]; r2 = t[1];
        t = __builtin_amdgcn_permlane32_swap(r1, r3, false, false); r1 = t[0]; r3 = t[1];
        t = __builtin_amdgcn_permlane16_swap(r0, r1, false, false); r0 = t[0]; r1 = t[1];
        t = __builtin_amdgcn_permlane16_swap(r2, r3, false, false); r2 = t[0]; r3 = t[1];
        v[0] = __uint_as_float(r0); v[1] = __uint_as_float(r1); v[2] = __uint_as_float(r2); v[3] = __uint_as_float(r3);
    };
    // One k step (j, i) at a time across all NYW accumulators, so that consecutive MFMAs never depend on each other; the
    // NYW values of B for a step are read from LDS one step ahead of the MFMAs that use them.
    auto multiply_half = [&](int unit, int c, int h) {
        int b_index = ((unit % p.parts) * NYW * KJ + c * TALL_CH + h * HALF) * 256 + lane;
        // (opaque per pass: with K == 96 the addresses never change and every B value would be hoisted into registers;
        // the index, not the pointer, so that the reads stay LDS reads)
        asm volatile("" : "+v"(b_index));
        const float* b0 = bfrag + b_index;
        constexpr int STEPS = HALF * 4;
        float b[2][NYW];
        auto read_b = [&](int t) {  // t = 4 jj + i
            const float* q = b0 + t * 64;
#pragma unroll
            for (int y = 0; y < NYW; ++y) b[t & 1][y] = q[(long)y * KJ * 256];
        };
        read_b(0);
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            const int j = h * HALF + t / 4, i = t % 4;
            if (i == 0) transpose_k(a[j]);
            if (t + 1 < STEPS) read_b(t + 1);
#pragma unroll
            for (int y = 0; y < NYW; ++y) acc[y] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[t & 1][y], a[j][i], acc[y], 0, 0, 0);
        }
    };
    const float* bias_lds = bfrag + p.K * p.N;
    // The finished unit, TALL_STORE: per 16-column tile one LDS read (bias), four additions, one 16-byte store.
    auto finish_store = [&](int unit) {
        const int row = 16 * (unit / p.parts) + li, col0 = 16 * NYW * (unit % p.parts) + 4 * g;
        if (row >= p.M) return;
        float* crow = p.C + (long)row * p.ldc + col0;
#pragma unroll
        for (int y = 0; y < NYW; ++y) {
            f4t v = acc[y];
            if (p.bias != nullptr) {
                const f4t bv = *reinterpret_cast<const f4t*>(bias_lds + col0 + 16 * y);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] + bv[e];
            }
            f4t* out = reinterpret_cast<f4t*>(crow + 16 * y);
            if (p.accumulate) {
                const f4t old = *out;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = old[e] + v[e];
            }
            *out = v;
        }
    };
    // The finished unit, TALL_GENERAL.  A runtime loop over its tiles (the activation code is there once, not once per
    // accumulator); the accumulators, and the values the upstream activation's derivative is taken of, rotate through
    // element 0 so that no register is indexed at run time.  Those values are fetched while the unit's last 96 columns are
    // multiplied.
    f4t src[NYW];
    auto fetch_src = [&](int unit) {
        const int row = min(16 * (unit / p.parts) + li, p.M - 1);
        const float* s0 = p.act_src + (long)row * p.ld_act + 16 * NYW * (unit % p.parts) + 4 * g;
#pragma unroll
        for (int y = 0; y < NYW; ++y) src[y] = *reinterpret_cast<const f4t*>(s0 + 16 * y);
    };
    auto finish_general = [&](int unit) {
        const int row = 16 * (unit / p.parts) + li, col0 = 16 * NYW * (unit % p.parts) + 4 * g;
        const bool live = row < p.M;
        const long crow = (long)row * p.ldc, zrow = (long)row * p.ldz;
#pragma unroll 1
        for (int y = 0; y < NYW; ++y) {
            const int col = col0 + 16 * y;
            f4t v = acc[0];
            const f4t sv = src[0];
#pragma unroll
            for (int k = 0; k + 1 < NYW; ++k) {
                acc[k] = acc[k + 1];
                src[k] = src[k + 1];
            }
            if (!live) continue;
            if (EPI != TALL_GELU_BWD && p.bias != nullptr) {
                const f4t bv = *reinterpret_cast<const f4t*>(bias_lds + col);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] + bv[e];
            }
            if (EPI != TALL_GELU_BWD && p.Z != nullptr) *reinterpret_cast<f4t*>(p.Z + zrow + col) = v;
            if (EPI == TALL_GELU_FWD) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = act_forward<float>(ACT_GELU, v[e], 0.f);
            } else if (EPI == TALL_GELU_BWD) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = v[e] * act_derivative<float>(ACT_GELU, sv[e], 0.f);
            } else {
                if (p.act_fwd != ACT_NONE) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = act_forward<float>(p.act_fwd, v[e], p.alpha);
                }
                if (p.act_bwd != ACT_NONE) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = v[e] * act_derivative<float>(p.act_bwd, sv[e], p.alpha);
                }
            }
            f4t* out = reinterpret_cast<f4t*>(p.C + crow + col);
            if (p.accumulate) {
                const f4t old = *out;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = old[e] + v[e];
            }
            *out = v;
        }
    };
    auto finish = [&](int unit) {
        if (EPI == TALL_STORE) finish_store(unit);
        else finish_general(unit);
    };
    auto zero = [&] {
#pragma unroll
        for (int y = 0; y < NYW; ++y) acc[y] = f4t{0.f, 0.f, 0.f, 0.f};
    };
    // One unit per pass.  The next unit's number is asked for at the top of the pass and read when the first loads for
    // it are due (half a chunk of MFMAs later).  With ONE_CHUNK the pass is straight-line code: a wait placed after a
    // branch around the stores would include them.
    int unit = first + wave;
#pragma unroll 1
    for (int pass = 0;; ++pass) {
        int ticket = 0;
        if (lane == 0) ticket = __hip_atomic_fetch_add(next_counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        int next_unit = unit;
        bool has_next = false;
        auto resolve = [&] {
            const int t = __builtin_amdgcn_readfirstlane(ticket);
            has_next = t < count;
            next_unit = has_next ? first + t : unit;  // (the last unit is fetched twice rather than branched around)
        };
        zero();
        if (ONE_CHUNK) {
            if (EPI == TALL_GELU_BWD || (EPI == TALL_GENERAL && p.act_bwd != ACT_NONE)) fetch_src(unit);
            multiply_half(unit, 0, 0);
            resolve();
            load_half(next_unit, 0, 0);
            multiply_half(unit, 0, 1);
            load_half(next_unit, 0, 1);
        } else {
#pragma unroll 1
            for (int c = 0; c < nchunks; ++c) {
                const bool last = c == nchunks - 1;
                if ((EPI == TALL_GELU_BWD || (EPI == TALL_GENERAL && p.act_bwd != ACT_NONE)) && last) fetch_src(unit);
                multiply_half(unit, c, 0);
                if (last) resolve();
                const int nu = last ? next_unit : unit, nc = last ? 0 : c + 1;
                load_half(nu, nc, 0);
                multiply_half(unit, c, 1);
                load_half(nu, nc, 1);
            }
        }
        finish(unit);
        if (!has_next) break;
        unit = next_unit;
    }
}

int tall_compute_units() {
    static const int v = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        return n;
    }();
    return v;
}

template <int NYW, int EPI, bool ONE_CHUNK>
hipError_t launch_variant(const TallArgs& k, unsigned grid, size_t lds, hipStream_t stream) {
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tall_kernel<NYW, EPI, ONE_CHUNK>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)TALL_MAX_LDS);
    if (attr != hipSuccess) return attr;
    hipLaunchKernelGGL((gemm_tall_kernel<NYW, EPI, ONE_CHUNK>), dim3(grid), dim3(TALL_THREADS), lds, stream, k);
    return hipGetLastError();
}
template <int NYW>
hipError_t launch_nyw(const TallArgs& k, unsigned grid, size_t lds, hipStream_t stream) {
    const bool general = k.Z != nullptr || k.act_fwd != ACT_NONE || k.act_bwd != ACT_NONE;
    const bool one = k.K == 16 * TALL_CH;
    if (k.act_fwd == ACT_GELU && k.act_bwd == ACT_NONE)
        return one ? launch_variant<NYW, TALL_GELU_FWD, true>(k, grid, lds, stream) : launch_variant<NYW, TALL_GELU_FWD, false>(k, grid, lds, stream);
    if (k.act_bwd == ACT_GELU && k.act_fwd == ACT_NONE && k.Z == nullptr && k.bias == nullptr)
        return one ? launch_variant<NYW, TALL_GELU_BWD, true>(k, grid, lds, stream) : launch_variant<NYW, TALL_GELU_BWD, false>(k, grid, lds, stream);
    if (general) return one ? launch_variant<NYW, TALL_GENERAL, true>(k, grid, lds, stream) : launch_variant<NYW, TALL_GENERAL, false>(k, grid, lds, stream);
    return one ? launch_variant<NYW, TALL_STORE, true>(k, grid, lds, stream) : launch_variant<NYW, TALL_STORE, false>(k, grid, lds, stream);
}

// Tiles per unit for a product of `ny` 16-column tiles: four, three or two, whichever divides ny first.  Narrow units
// keep the epilogue's registers few (the general one holds a second value per accumulator) and give every matrix core
// many units, so that their shares differ by little; wider ones (six, eight, nine tiles; six again with the lane-group
// transposes in place, which a wider unit shares among more MFMAs) were measured no faster for the plain store and up to
// 40 % slower for the general epilogue.
int tall_unit_tiles(int64_t ny) {
    static const int forced = [] { const char* e = getenv("PRAD_GEMM_TALL_UNIT_TILES"); return e ? atoi(e) : 0; }();  // tuning aid
    for (int w : {4, 3, 2})
        if (forced == w && ny % w == 0) return w;
    for (int w : {4, 3, 2})
        if (ny % w == 0) return w;
    return 0;
}

bool aligned16(const void* q, int64_t ld) { return q == nullptr || (reinterpret_cast<uintptr_t>(q) % 16 == 0 && ld % 4 == 0); }

}  // namespace

// Shapes that go to the kernel above: float, A not transposed, one product, at least TALL_MIN_ROWS rows, K a multiple of
// 96 and N a multiple of 32 or 48 with K * N floats within 144 KB, every row 16-byte aligned.
// PRAD_GEMM_TALL=0 switches it off (a tuning aid).
bool gemm_tall_eligible(const GemmArgs<float>& a) {
    static const bool enabled = [] { const char* e = getenv("PRAD_GEMM_TALL"); return !(e && e[0] == '0'); }();
    static const int64_t min_rows = [] { const char* e = getenv("PRAD_GEMM_TALL_MIN_ROWS"); return e ? (int64_t)atoll(e) : TALL_MIN_ROWS; }();
    if (!enabled || a.transA || a.batch != 1 || a.batch_inner > 1 || a.nseg > 1 || a.tile_sums != nullptr || a.colsum_dst != nullptr ||
        a.lstm_hidden != 0)
        return false;
    if (a.M < min_rows || a.M >= (1 << 27) || a.K < 16 * TALL_CH || a.K % (16 * TALL_CH) != 0 || a.N % 16 != 0) return false;
    if (tall_unit_tiles(a.N / 16) == 0) return false;
    if ((size_t)a.K * a.N * sizeof(float) > TALL_MAX_B) return false;
    if (!aligned16(a.A, a.lda) || !aligned16(a.B, a.ldb) || !aligned16(a.C, a.ldc) || !aligned16(a.Z, a.ldz) ||
        !aligned16(a.act_src, a.ld_act) || !aligned16(a.bias, 4))
        return false;
    if (a.lda >= (1 << 20)) return false;  // (a lane's byte offset into A is kept in 32 bits: rows * lda * 4 < 2^32 is checked at launch)
    return true;
}

hipError_t launch_gemm_tall(const GemmArgs<float>& a, hipStream_t stream) {
    if (!gemm_tall_eligible(a) || (uint64_t)a.M * (uint64_t)a.lda * 4u >= ((uint64_t)1 << 32)) return hipErrorNotSupported;
    TallArgs k{};
    k.A = a.A; k.B = a.B; k.C = a.C; k.bias = a.bias; k.Z = a.Z; k.act_src = a.act_src;
    k.lda = a.lda; k.ldb = a.ldb; k.ldc = a.ldc; k.ldz = a.ldz; k.ld_act = a.ld_act;
    k.M = (int)a.M; k.N = (int)a.N; k.K = (int)a.K;
    k.transB = a.transB; k.accumulate = a.accumulate; k.act_fwd = a.act_fwd; k.act_bwd = a.act_bwd; k.alpha = a.alpha;
    k.blocks = (int)((a.M + 15) / 16);
    const int nyw = tall_unit_tiles(a.N / 16);
    k.parts = (int)(a.N / 16) / nyw;
    const unsigned grid = (unsigned)std::min<int64_t>(tall_compute_units(), (int64_t)k.blocks * k.parts);
    const size_t lds = ((size_t)a.K * a.N + (size_t)a.N + 4) * sizeof(float);  // B as fragments, the bias, the unit counter
    switch (nyw) {
        case 2: return launch_nyw<2>(k, grid, lds, stream);
        case 3: return launch_nyw<3>(k, grid, lds, stream);
        case 4: return launch_nyw<4>(k, grid, lds, stream);
        default: return hipErrorNotSupported;
    }
}

}  // namespace prad
