// dB = A^T . dC for a very long K and a small output (float): the weight gradient of a layer of a few hundred inputs and
// outputs applied to tens of thousands of rows (96 x 288 from K = 50 176 rows in a windowed-attention block),
// MatrixMultiplyOperation.Backward (src/RMAD/MatrixMultiplyOperation.cs:88-126), with the bias gradient - the column
// sums of dC, MatrixAddBroadcastingOperation.Backward (src/RMAD/MatrixAddBroadcastingOperation.cs:57-70) - taken from
// the same pass over dC when asked for.  On the tiled kernels such a product is split along K into 32 x 32 tiles: a
// wavefront's 16 x 16 share takes two LDS reads per MFMA and the LDS pipe bounds it at about 40 % of the matrix cores,
// every tile column re-reads its panel of A and every tile row its panel of dC, and the column sums are two more
// launches over dC.  Here the split is along K only:
//
//   * a workgroup takes a contiguous range of K (slabs of 16 rows of A and dC) and multiplies it into the WHOLE M x N
//     output: its four or eight wavefronts hold up to 18 tiles of 16 x 16 each in their accumulators, so a k step reads
//     RT + CT fragments for RT x CT MFMAs (8 for 15 at 96 x 288) and A and dC are read from memory exactly once;
//   * the transfers of the slabs ahead and the next k step's fragment reads are issued between the MFMAs, as in the tiled
//     kernels' main loop; the MFMA code is straight-line (tile counts are template arguments, tiles past M or N multiply
//     zeros kept in LDS);
//   * each workgroup writes its partial M x N (and its partial column sums, accumulated in double) to the workspace and a
//     second launch adds the partials in workgroup order: deterministic, two-level summation along K.
#include "common.h"

#include <cstdlib>
#include <type_traits>

namespace prad {

namespace {

typedef float f4s __attribute__((ext_vector_type(4)));
constexpr int SK_KB = 16;  // rows of K per slab
// LDS pitch of a slab row, in floats: = 16 (mod 64), so that the four rows (k) of a fragment read fall into different
// banks for 16 consecutive columns, and a multiple of 4.
__host__ __device__ constexpr int sk_pitch(int x) { return x + ((16 - x % 64 + 64) % 64); }

template <int RT, int CT, int WR, int WC>
struct SkShape {
    static constexpr int THREADS = 64 * WR * WC;                // four or eight wavefronts, WR x WC over the output
    static constexpr int MP = 16 * RT * WR, NP = 16 * CT * WC;  // the output padded to whole tiles of the wavefront grid
    static constexpr int PA = sk_pitch(MP), PB = sk_pitch(NP);
    static constexpr int NVA = (SK_KB * MP / 4 + THREADS - 1) / THREADS;  // 16-byte vectors per thread and slab
    static constexpr int NVB = (SK_KB * NP / 4 + THREADS - 1) / THREADS;
    static constexpr int NCS = (NP + THREADS - 1) / THREADS;              // columns of dC per thread for the column sums
    static constexpr int STAGE = SK_KB * (PA + PB);
};

struct SkArgs {
    const float* A; int64_t lda;  // K x M as stored
    const float* B; int64_t ldb;  // K x N as stored (dC)
    float* partial;               // workgroups x M x N
    double* colsum_partial;       // workgroups x N, or nullptr
    int M, N;
    int64_t slabs;                // K / SK_KB
    int slabs_per_wg;
};

// Eight wavefronts where the output has more than 36 tiles for four: two per SIMD with at most 18 tiles each keep the
// accumulators in the 128 registers a lane then has and overlap one another's waits; with four wavefronts of up to 36
// tiles the compiler keeps part of the accumulators in the other register file and copies them in and out around the
// loop (measured: 45 to 55 us for 21 us of MFMAs).
template <int RT, int CT, int WR, int WC>
__global__ void __launch_bounds__(64 * WR * WC, WR * WC == 4 ? 2 : 1) gemm_skinny_kernel(const SkArgs p) {
    typedef SkShape<RT, CT, WR, WC> S;
    constexpr int SK_THREADS = S::THREADS;
    constexpr int PA = S::PA, PB = S::PB, NVA = S::NVA, NVB = S::NVB;
    const int M = p.M, N = p.N;
    // (the wavefront index as a scalar, so that what derives from it steers scalar branches)
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), wr = wave / WC, wc = wave % WC;
    const int li = lane & 15, g = lane >> 4;
    __shared__ __attribute__((aligned(16))) float lds[2 * S::STAGE + 4];  // [stage][A slab | B slab], and a slot for the vectors of threads that have none to move

    // zeros once: the columns past M and N are never written again
    for (int i = tid; i < 2 * S::STAGE; i += SK_THREADS) lds[i] = 0.f;

    // this thread's vectors of a slab: byte offset from the slab's first row in memory, float offset inside the stage (-1: none)
    int offA[NVA], dstA[NVA], offB[NVB], dstB[NVB];
#pragma unroll
    for (int e = 0; e < NVA; ++e) {
        const int v = e * SK_THREADS + tid, per_row = M / 4;
        const bool ok = v < SK_KB * per_row;
        offA[e] = ok ? (int)(((int64_t)(v / per_row) * p.lda + (v % per_row) * 4) * 4) : 0;
        dstA[e] = ok ? (v / per_row) * PA + (v % per_row) * 4 : -1;  // (-1: goes to the spare slot; no branch between the MFMAs)
    }
#pragma unroll
    for (int e = 0; e < NVB; ++e) {
        const int v = e * SK_THREADS + tid, per_row = N / 4;
        const bool ok = v < SK_KB * per_row;
        offB[e] = ok ? (int)(((int64_t)(v / per_row) * p.ldb + (v % per_row) * 4) * 4) : 0;
        dstB[e] = ok ? (v / per_row) * PB + (v % per_row) * 4 : -1;
    }
    const int64_t slab0 = (int64_t)blockIdx.x * p.slabs_per_wg;
    const int nsl = (int)min((int64_t)p.slabs_per_wg, p.slabs - slab0);

    f4s acc[RT][CT];
#pragma unroll
    for (int x = 0; x < RT; ++x)
#pragma unroll
        for (int y = 0; y < CT; ++y) acc[x][y] = f4s{0.f, 0.f, 0.f, 0.f};
    double cs[S::NCS];  // column sums of dC over this workgroup's rows: columns tid, tid + threads, ...
#pragma unroll
    for (int h = 0; h < S::NCS; ++h) cs[h] = 0.0;

    f4s ra[2][NVA], rb[2][NVB];
    auto slab_a = [&](int s) { return p.A + (slab0 + min(s, nsl - 1)) * SK_KB * p.lda; };  // (past the range: the last slab again, never used)
    auto slab_b = [&](int s) { return p.B + (slab0 + min(s, nsl - 1)) * SK_KB * p.ldb; };
    auto load_vec = [](const float* base, int off) {
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, -1, 0x00020000);
        return __builtin_bit_cast(f4s, __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0));
    };
    // op o of a slab's transfers: even o = vector o/2 of the set `from` into stage `to`; odd o = vector o/2 of slab `s` from memory into set `into`
    auto transfer = [&](int o, auto from_c, float* __restrict__ to, auto into_c, int s) {
        constexpr int from = decltype(from_c)::value, into = decltype(into_c)::value;
        const int j = o >> 1;
        if (o & 1) {
            if (j < NVA) ra[into][j] = load_vec(slab_a(s), offA[j]);
            else rb[into][j - NVA] = load_vec(slab_b(s), offB[j - NVA]);
        } else {
            if (j < NVA) *reinterpret_cast<f4s*>(dstA[j] >= 0 ? to + dstA[j] : lds + 2 * S::STAGE) = ra[from][j];
            else *reinterpret_cast<f4s*>(dstB[j - NVA] >= 0 ? to + SK_KB * PA + dstB[j - NVA] : lds + 2 * S::STAGE) = rb[from][j - NVA];
        }
    };
    constexpr int NOPS = 2 * (NVA + NVB), NM = RT * CT, NR = RT + CT, KSTEPS = SK_KB / 4, SLOTS = KSTEPS * NM;
    // One slab of MFMAs from `st`, the transfers `op(o)` and the next k step's fragment reads issued between them.
    auto compute = [&](const float* __restrict__ st, auto&& op) {
        const float* __restrict__ sA = st + wr * RT * 16 + li;
        const float* __restrict__ sB = st + SK_KB * PA + wc * CT * 16 + li;
        float a[2][RT], b[2][CT];
        auto read = [&](int s, int r) {
            const int k = 4 * s + g;
            if (r < RT) a[s & 1][r] = sA[k * PA + 16 * r];
            else b[s & 1][r - RT] = sB[k * PB + 16 * (r - RT)];
        };
#pragma unroll
        for (int r = 0; r < NR; ++r) read(0, r);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                const int x = m / CT, y = m % CT;
                acc[x][y] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s & 1][x], b[s & 1][y], acc[x][y], 0, 0, 0);
                if (s + 1 < KSTEPS) {
#pragma unroll
                    for (int r = m * NR / NM; r < (m + 1) * NR / NM; ++r) read(s + 1, r);
                }
                const int q = s * NM + m;
#pragma unroll
                for (int o = q * NOPS / SLOTS; o < (q + 1) * NOPS / SLOTS; ++o) op(o);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    // column sums of the dC slab in `st` (rows of K in ascending order, accumulated in double)
    auto colsum = [&](const float* __restrict__ st) {
        if (p.colsum_partial == nullptr) return;
        const float* __restrict__ sB = st + SK_KB * PA;
#pragma unroll
        for (int h = 0; h < S::NCS; ++h) {
            const int j = tid + h * SK_THREADS;
            if (j < N) {
#pragma unroll
                for (int k = 0; k < SK_KB; ++k) cs[h] += (double)sB[k * PB + j];
            }
        }
    };
    std::integral_constant<int, 0> c0;
    std::integral_constant<int, 1> c1;

    if (nsl > 0) {
#pragma unroll
        for (int o = 1; o < NOPS; o += 2) transfer(o, c0, lds, c0, 0);  // slab 0 -> set 0
#pragma unroll
        for (int o = 1; o < NOPS; o += 2) transfer(o, c0, lds, c1, 1);  // slab 1 -> set 1
        __syncthreads();                                                 // (the zero fill is done)
#pragma unroll
        for (int o = 0; o < NOPS; o += 2) transfer(o, c0, lds, c0, 0);  // set 0 -> stage 0
        __syncthreads();
        // (no branch inside the loop body: a branch around a slab's MFMAs sends all accumulators through copies at every
        // iteration; an odd last slab is multiplied after the loop)
        int s = 0;
        for (; s + 1 < nsl; s += 2) {
            // stage 0 holds slab s, set 1 slab s+1; slab s+2 goes into set 0
            colsum(lds);
            compute(lds, [&](int o) { transfer(o, c1, lds + S::STAGE, c0, s + 2); });
            __syncthreads();
            // stage 1 holds slab s+1, set 0 slab s+2; slab s+3 goes into set 1
            colsum(lds + S::STAGE);
            compute(lds + S::STAGE, [&](int o) { transfer(o, c0, lds, c1, s + 3); });
            __syncthreads();
        }
        if (s < nsl) {
            colsum(lds);
            compute(lds, [](int) {});
        }
    }
    // this workgroup's partial output and column sums
    float* __restrict__ out = p.partial + (int64_t)blockIdx.x * M * N;
#pragma unroll
    for (int x = 0; x < RT; ++x)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int i = (wr * RT + x) * 16 + 4 * g + r;
#pragma unroll
            for (int y = 0; y < CT; ++y) {
                const int j = (wc * CT + y) * 16 + li;
                if (i < M && j < N) out[(int64_t)i * N + j] = acc[x][y][r];
            }
        }
    if (p.colsum_partial != nullptr) {
#pragma unroll
        for (int h = 0; h < S::NCS; ++h) {
            const int j = tid + h * SK_THREADS;
            if (j < N) p.colsum_partial[(int64_t)blockIdx.x * N + j] = cs[h];
        }
    }
}

// Adds the workgroups' partial outputs (and column sums) in a fixed order: sixteen threads per element each add every
// sixteenth partial, in ascending order, sixteen loads in flight at a time, and their sums are added in thread order (one
// thread walking all partials of an element was a chain of some 250 dependent loads: 110 us).
constexpr int SKR_WAYS = 16, SKR_ELEMS = 256 / SKR_WAYS;
__global__ void __launch_bounds__(256) skinny_reduce_kernel(const float* __restrict__ partial, const double* __restrict__ colsum_partial,
                                                            float* __restrict__ C, int64_t ldc, float* __restrict__ colsum_dst, int M, int N,
                                                            int parts, int accumulate) {
    __shared__ double red[256];
    const int64_t total = (int64_t)M * N;                                // (a multiple of 4: N is)
    const int q = threadIdx.x / SKR_ELEMS, e = threadIdx.x % SKR_ELEMS;  // way; element of the block (four consecutive outputs)
    const int64_t blocks_c = (total / 4 + SKR_ELEMS - 1) / SKR_ELEMS;
    if ((int64_t)blockIdx.x < blocks_c) {
        const int64_t idx = ((int64_t)blockIdx.x * SKR_ELEMS + e) * 4;
        f4s v = {0.f, 0.f, 0.f, 0.f};
        if (idx < total) {
            for (int w = q; w < parts; w += 16 * SKR_WAYS) {
                f4s t[16];
#pragma unroll
                for (int u = 0; u < 16; ++u)
                    t[u] = w + u * SKR_WAYS < parts ? *reinterpret_cast<const f4s*>(partial + (int64_t)(w + u * SKR_WAYS) * total + idx) : f4s{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int u = 0; u < 16; ++u)
                    if (w + u * SKR_WAYS < parts) v = v + t[u];
            }
        }
        __shared__ f4s red4[256];
        red4[threadIdx.x] = v;
        __syncthreads();
        if (q == 0 && idx < total) {
            f4s sum = red4[e];
#pragma unroll
            for (int u = 1; u < SKR_WAYS; ++u) sum = sum + red4[u * SKR_ELEMS + e];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float* c = C + ((idx + i) / N) * ldc + (idx + i) % N;
                *c = accumulate ? *c + sum[i] : sum[i];
            }
        }
    } else if (colsum_dst != nullptr) {
        const int64_t j = ((int64_t)blockIdx.x - blocks_c) * SKR_ELEMS + e;
        double v = 0.0;
        if (j < N) {
            for (int w = q; w < parts; w += 16 * SKR_WAYS) {  // (sixteen loads in flight, added in ascending order)
                double t[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) t[u] = w + u * SKR_WAYS < parts ? colsum_partial[(int64_t)(w + u * SKR_WAYS) * N + j] : 0.0;
#pragma unroll
                for (int u = 0; u < 16; ++u)
                    if (w + u * SKR_WAYS < parts) v += t[u];
            }
        }
        red[threadIdx.x] = v;
        __syncthreads();
        if (q == 0 && j < N) {
            double sum = red[e];
#pragma unroll
            for (int u = 1; u < SKR_WAYS; ++u) sum += red[u * SKR_ELEMS + e];
            colsum_dst[j] = (float)sum;
        }
    }
}

struct SkClass { int rt, ct, wr, wc; };
// tiles per wavefront (rows, columns) and the wavefront grid: 96 x 96, 96 x 320, 96 x 384, 384 x 96 outputs at most
constexpr SkClass SK_CLASSES[] = {{3, 3, 2, 2}, {3, 5, 2, 4}, {3, 6, 2, 4}, {3, 6, 8, 1}};

int sk_class_of(int64_t M, int64_t N) {
    for (int i = 0; i < (int)(sizeof(SK_CLASSES) / sizeof(SK_CLASSES[0])); ++i) {
        const SkClass& c = SK_CLASSES[i];
        if (M <= 16 * c.rt * c.wr && N <= 16 * c.ct * c.wc) return i;
    }
    return -1;
}
int sk_compute_units() {
    static const int v = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        return n;
    }();
    return v;
}
// Slabs per workgroup and workgroups.
void sk_plan(int64_t K, int* slabs_per_wg, int* wgs) {
    const int64_t slabs = K / SK_KB;
    const int64_t per = (slabs + sk_compute_units() - 1) / sk_compute_units();
    *slabs_per_wg = (int)per;
    *wgs = (int)((slabs + per - 1) / per);
}

}  // namespace

// Shapes that go to the kernel above: float, A^T . B with both operands row-major K x M and K x N, K a multiple of 16 and
// at least 4096 rows, the output at most 96 x 384 or 384 x 96, every row 16-byte aligned, no epilogue but accumulation.
// A column sum may ride along if it is that of the second operand.  PRAD_GEMM_SKINNY=0 switches it off (tuning aid).
bool gemm_skinny_eligible(const GemmArgs<float>& a) {
    static const bool enabled = [] { const char* e = getenv("PRAD_GEMM_SKINNY"); return !(e && e[0] == '0'); }();
    static const int64_t min_k = [] { const char* e = getenv("PRAD_GEMM_SKINNY_MIN_K"); return e ? (int64_t)atoll(e) : (int64_t)4096; }();
    if (!enabled || !a.transA || a.transB || a.batch != 1 || a.batch_inner > 1 || a.nseg > 1 || a.tile_sums != nullptr) return false;
    if (a.bias != nullptr || a.Z != nullptr || a.act_fwd != ACT_NONE || a.act_bwd != ACT_NONE) return false;
    if (a.K < min_k || a.K % SK_KB != 0 || a.M < 16 || a.N < 16 || a.M % 4 != 0 || a.N % 4 != 0 || sk_class_of(a.M, a.N) < 0) return false;
    if (a.lda % 4 != 0 || a.ldb % 4 != 0 || reinterpret_cast<uintptr_t>(a.A) % 16 != 0 || reinterpret_cast<uintptr_t>(a.B) % 16 != 0) return false;
    if (a.lda >= (1 << 20) || a.ldb >= (1 << 20)) return false;  // (byte offsets inside a slab are kept in 32 bits)
    if (a.colsum_dst != nullptr && (a.colsum_src != a.B || a.colsum_rows != a.K || a.colsum_cols != a.N)) return false;
    return true;
}
size_t gemm_skinny_workspace_bytes(const GemmArgs<float>& a) {
    if (!gemm_skinny_eligible(a)) return 0;
    int per, wgs;
    sk_plan(a.K, &per, &wgs);
    return (size_t)wgs * ((size_t)a.M * a.N * sizeof(float) + (size_t)a.N * sizeof(double)) + 256;
}

hipError_t launch_gemm_skinny(const GemmArgs<float>& a, hipStream_t stream) {
    if (a.split_ws == nullptr || !gemm_skinny_eligible(a)) return hipErrorNotSupported;
    SkArgs k{};
    k.A = a.A; k.lda = a.lda; k.B = a.B; k.ldb = a.ldb; k.M = (int)a.M; k.N = (int)a.N; k.slabs = a.K / SK_KB;
    int wgs;
    sk_plan(a.K, &k.slabs_per_wg, &wgs);
    k.partial = a.split_ws;
    // (the column sums' partials lie after the outputs', 8-byte aligned)
    const size_t pbytes = ((size_t)wgs * a.M * a.N * sizeof(float) + 7) & ~(size_t)7;
    k.colsum_partial = a.colsum_dst != nullptr ? reinterpret_cast<double*>(reinterpret_cast<char*>(a.split_ws) + pbytes) : nullptr;
    const dim3 grid((unsigned)wgs);
    switch (sk_class_of(a.M, a.N)) {
        case 0: hipLaunchKernelGGL((gemm_skinny_kernel<3, 3, 2, 2>), grid, dim3(256), 0, stream, k); break;
        case 1: hipLaunchKernelGGL((gemm_skinny_kernel<3, 5, 2, 4>), grid, dim3(512), 0, stream, k); break;
        case 2: hipLaunchKernelGGL((gemm_skinny_kernel<3, 6, 2, 4>), grid, dim3(512), 0, stream, k); break;
        case 3: hipLaunchKernelGGL((gemm_skinny_kernel<3, 6, 8, 1>), grid, dim3(512), 0, stream, k); break;
        default: return hipErrorNotSupported;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int64_t blocks = ((int64_t)a.M * a.N / 4 + SKR_ELEMS - 1) / SKR_ELEMS + (a.colsum_dst != nullptr ? (a.N + SKR_ELEMS - 1) / SKR_ELEMS : 0);
    hipLaunchKernelGGL(skinny_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, k.partial, k.colsum_partial, a.C, a.ldc,
                       a.colsum_dst, (int)a.M, (int)a.N, wgs, a.accumulate);
    return hipGetLastError();
}

}  // namespace prad
