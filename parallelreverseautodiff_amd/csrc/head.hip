// The last layer of a classifier with its loss, forward and backward, in one launch: MatrixMultiplyOperation.Forward
// (src/RMAD/MatrixMultiplyOperation.cs:50-80) and MatrixAddBroadcastingOperation.Forward of the output layer,
// SoftmaxOperation.Forward (src/RMAD/SoftmaxOperation.cs:45-110), CategoricalCrossEntropyLossOperation.Forward and
// Backward (src/RMAD/Loss/CategoricalCrossEntropyLossOperation.cs:37-86), SoftmaxOperation.Backward, then the layer's
// Backward: bias gradient, dW = A^T . dZ, dA = dZ . W^T with the activation Backward of the layer below.
//
// For a batch of a few dozen rows and a few dozen classes these are seven dependent steps of almost no work; as separate
// launches each costs a launch's latency.  Here one workgroup holds the layer's input, its weights and the class rows
// in LDS and walks through the steps with workgroup barriers between them.
//
// Bits: every value equals what the separate launches give.  The three products run on the matrix cores with the same
// instruction and the same assignment of k to its steps as the tiled kernels (k = 4 s + lane / 16, s ascending; operands
// past an edge are zeros, which add nothing); softmax, cross-entropy and the column sums are the statements of
// csrc/loss.hip and colsum_block, with the wavefront reductions cut down to the lanes that hold a row (the other lanes
// of the wide reduction contribute exact zeros).  Where the separate path would split a product along K, or fold a float
// sum beyond K = 512, the order of that sum differs and the results agree to rounding instead.
#include "common.h"

#include <cstdlib>

namespace prad {

namespace {

constexpr int HEAD_THREADS = 1024, HEAD_WAVES = HEAD_THREADS / 64;
constexpr int DA_TILES = 2;  // tiles of dA per wavefront and round
constexpr size_t HEAD_MAX_LDS = 144 * 1024;

__host__ __device__ constexpr int round16(int x) { return (x + 15) / 16 * 16; }

template <typename T>
struct HeadLayout {
    int B16, H16, C16;
    int HP;  // pitch of the input block [B16][HP]: odd, so that lanes walking down a column fall on distinct banks
    int CP;  // pitch of the class rows and of the rows of W: odd as well
    size_t off_A, off_W, off_Z, off_D, off_T, off_bias, elems;  // element offsets
    size_t off_part, bytes;                                     // byte offsets
    __host__ __device__ HeadLayout(int B, int H, int C) {
        B16 = round16(B); H16 = round16(H); C16 = round16(C);
        HP = H16 + 1;
        CP = C16 + 1;
        off_A = 0;
        off_W = off_A + (size_t)B16 * HP;
        off_Z = off_W + (size_t)H16 * CP;
        off_D = off_Z + (size_t)B16 * CP;
        off_T = off_D + (size_t)B16 * CP;
        off_bias = off_T + (size_t)B16 * CP;
        elems = off_bias + (size_t)CP;
        off_part = (elems * sizeof(T) + 15) / 16 * 16;
        bytes = off_part + (4 + 256) * sizeof(double);
    }
};

typedef double d4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));
template <typename T> struct HeadMfma;
template <> struct HeadMfma<double> {
    typedef d4 Acc;
    typedef double Vec __attribute__((ext_vector_type(2)));
    static constexpr int VEC = 2;
    static __device__ __forceinline__ Acc mfma(double a, double b, Acc c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ int row(int r, int g) { return 4 * r + g; }
};
template <> struct HeadMfma<float> {
    typedef f4 Acc;
    typedef f4 Vec;
    static constexpr int VEC = 4;
    static __device__ __forceinline__ Acc mfma(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ int row(int r, int g) { return 4 * g + r; }
};

// A workgroup barrier that orders LDS accesses only: the waves exchange nothing through memory, and a full
// __syncthreads() would also wait for every global store issued so far (a round trip to memory per phase).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

__device__ __forceinline__ double max_of(double a, double b) { return fmax(a, b); }
__device__ __forceinline__ float max_of(float a, float b) { return fmaxf(a, b); }

// Sum / maximum over the `seg` lanes (16, 32 or 64) that hold one row, lanes past the row holding 0 / -inf: the values of
// wave_sum_t / wave_max_t over 64 lanes with one row per wavefront.  There the first steps add the zeros of the lanes
// beyond `seg` (which turns a -0 into +0: the addition of +0 below does the same), the rest are these steps.
template <typename T>
__device__ __forceinline__ T seg_sum(T v, int seg) {
    if (seg < 64) v = v + (T)0;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        if (off < seg) v += __shfl_xor(v, off, 64);
    return v;
}
template <typename T>
__device__ __forceinline__ T seg_max(T v, int seg) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        if (off < seg) v = max_of(v, __shfl_xor(v, off, 64));
    return v;
}

template <typename T>
__global__ void __launch_bounds__(HEAD_THREADS) classifier_head_kernel(const HeadArgs<T> p) {
    typedef HeadMfma<T> MF;
    typedef typename MF::Acc Acc;
    typedef typename MF::Vec Vec;
    constexpr int VEC = MF::VEC;
    extern __shared__ __attribute__((aligned(16))) unsigned char head_lds[];
    const int B = p.B, H = p.H, C = p.C;
    const HeadLayout<T> L(B, H, C);
    T* const lds = reinterpret_cast<T*>(head_lds);
    T* const sA = lds + L.off_A;        // the layer's input, [B16][HP], zeros past B and H
    T* const sW = lds + L.off_W;        // weights, [H16][CP], zeros past H and C
    T* const sZ = lds + L.off_Z;        // pre-activations, [B16][CP]
    T* const sD = lds + L.off_D;        // dZ, [B16][CP], zeros past B and C
    T* const sT = lds + L.off_T;        // targets, then the elements' terms of the loss
    T* const sBias = lds + L.off_bias;  // bias row
    double* const part = reinterpret_cast<double*>(head_lds + L.off_part);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, g = lane >> 4;

    // ---- everything that comes from memory is asked for at once; the first round of it before LDS is cleared ----
    // The values the lower activation's derivative is taken of, for the first two tiles of dA this wavefront will form
    // (used last).  Tiles of dA are numbered row tile first; wavefront w takes tiles w, w + 16 of every 32.
    const int tilesH = L.H16 / 16, tiles_dA = (L.B16 / 16) * tilesH;
    const bool with_act = p.dA != nullptr && p.act != ACT_NONE;
    T src[DA_TILES][4];
    auto fetch_src = [&](int first_tile) {
#pragma unroll
        for (int q = 0; q < DA_TILES; ++q) {
            const int t = first_tile + HEAD_WAVES * q;
            const int k = (t % tilesH) * 16 + li;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = (t / tilesH) * 16 + MF::row(r, g);
                src[q][r] = (with_act && t < tiles_dA && i < B && k < H) ? p.act_src[(long)i * H + k] : (T)0;
            }
        }
    };
    // A: a wavefront copies whole rows (row = wave + 16 rb, a lane one 16-byte vector of every 64); W and the targets: element
    // by element into their padded rows ((row, column) of an element from a float reciprocal: exact for these counts).
    const bool vec_A = H % VEC == 0 && reinterpret_cast<uintptr_t>(p.A) % 16 == 0;
    const int per_row = H / VEC, ncb = (per_row + 63) / 64;
    const int items_A = vec_A ? ((B + HEAD_WAVES - 1) / HEAD_WAVES) * ncb : 0;
    const float inv_C = 1.0f / (float)C;
    constexpr int ROUND = 4;  // loads in flight per thread and operand
    Vec av[ROUND];
    T wv[ROUND], tv[ROUND];
    auto item_A = [&](int q, int& row, int& vec) {
        const int rb = q / ncb;  // (wavefront-uniform)
        row = wave + HEAD_WAVES * rb;
        vec = lane + 64 * (q - rb * ncb);
        return q < items_A && row < B && vec < per_row;
    };
    auto load_round = [&](int round) {
#pragma unroll
        for (int u = 0; u < ROUND; ++u) {
            int row, vec;
            if (item_A(round * ROUND + u, row, vec)) av[u] = *reinterpret_cast<const Vec*>(p.A + row * H + vec * VEC);
            const int v = tid + (round * ROUND + u) * HEAD_THREADS;
            if (v < H * C) wv[u] = p.W[v];
            if (v < B * C) tv[u] = p.target[v];
        }
    };
    auto store_round = [&](int round) {
#pragma unroll
        for (int u = 0; u < ROUND; ++u) {
            int row, vec;
            if (item_A(round * ROUND + u, row, vec)) {
                T* dst = sA + row * L.HP + vec * VEC;
#pragma unroll
                for (int e = 0; e < VEC; ++e) dst[e] = av[u][e];
            }
            const int v = tid + (round * ROUND + u) * HEAD_THREADS;
            const int r = (int)(((float)v + 0.5f) * inv_C), o = r * L.CP + (v - r * C);
            if (v < H * C) sW[o] = wv[u];
            if (v < B * C) sT[o] = tv[u];
        }
    };
    const int most = max(max(items_A * HEAD_THREADS, H * C), B * C), rounds = (most + ROUND * HEAD_THREADS - 1) / (ROUND * HEAD_THREADS);
    load_round(0);
    fetch_src(wave);
    const T bias_c = (p.bias != nullptr && tid < C) ? p.bias[tid] : (T)0;

    for (int e = tid; e < (int)L.elems; e += HEAD_THREADS) lds[e] = (T)0;
    lds_barrier();
    store_round(0);
    for (int round = 1; round < rounds; ++round) {
        load_round(round);
        store_round(round);
    }
    if (!vec_A)
        for (int e = tid; e < B * H; e += HEAD_THREADS) sA[(e / H) * L.HP + e % H] = p.A[e];
    if (tid < C) sBias[tid] = bias_c;
    lds_barrier();

    // One tile's chain of MFMA steps, operands read from LDS four steps at a time (the step count is a multiple of four).
    // (Reading a group ahead of the MFMAs that use it was measured slower: the chain of dependent MFMAs is what a tile
    // lasts.)
    auto chain = [&](const T* a, int astep, const T* b, int bstep, int steps) {
        Acc acc = {0, 0, 0, 0};
        for (int s = 0; s < steps; s += 4) {
            const T a0 = a[0], a1 = a[astep], a2 = a[2 * astep], a3 = a[3 * astep];
            const T b0 = b[0], b1 = b[bstep], b2 = b[2 * bstep], b3 = b[3 * bstep];
            acc = MF::mfma(a0, b0, acc);
            acc = MF::mfma(a1, b1, acc);
            acc = MF::mfma(a2, b2, acc);
            acc = MF::mfma(a3, b3, acc);
            a += 4 * astep; b += 4 * bstep;
        }
        return acc;
    };

    // ---- Z = A . W + bias ----
    {
        const int tilesC = L.C16 / 16, tiles = (L.B16 / 16) * tilesC;
        for (int t = wave; t < tiles; t += HEAD_WAVES) {
            const int i0 = (t / tilesC) * 16, c0 = (t % tilesC) * 16;
            const Acc acc = chain(sA + (i0 + li) * L.HP + g, 4, sW + g * L.CP + c0 + li, 4 * L.CP, L.H16 / 4);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = i0 + MF::row(r, g), c = c0 + li;
                if (i < B && c < C) {
                    T v = acc[r];
                    if (p.bias != nullptr) v = v + sBias[c];
                    if (p.Z != nullptr) p.Z[(long)i * C + c] = v;
                    sZ[i * L.CP + c] = v;
                }
            }
        }
    }
    lds_barrier();

    // ---- softmax, the loss gradient and the softmax gradient, a row per `seg` lanes ----
    {
        const int seg = C <= 16 ? 16 : C <= 32 ? 32 : 64;
        const int rows_per_wave = 64 / seg, c = lane % seg;
        const T scale = (T)1 / (T)B;
        for (int r0 = 0; r0 < B; r0 += HEAD_WAVES * rows_per_wave) {
            const int i = r0 + wave * rows_per_wave + lane / seg;
            const bool on = c < C && i < B;
            const T xv = on ? sZ[i * L.CP + c] : (T)0;
            const T m = seg_max<T>(on ? xv : (T)-INFINITY, seg);
            const T e = on ? short_exp(xv - m) : (T)0;
            const T s = seg_sum<T>(e, seg);
            const T pr = e / s;
            const T gr = on ? -scale * sT[i * L.CP + c] / (pr + (T)1e-15) : (T)0;
            const T dot = seg_sum<T>(on ? gr * pr : (T)0, seg);
            if (on) {
                const T dz = pr * (gr - dot);
                p.P[i * C + c] = pr;
                p.dP[i * C + c] = gr;
                p.dZ[i * C + c] = dz;
                sD[i * L.CP + c] = dz;
                // the element's term of the loss, added up below; it takes the target's place
                if (p.loss != nullptr) sT[i * L.CP + c] = -sT[i * L.CP + c] * (T)log((double)(pr + (T)1e-15));
            }
        }
    }
    lds_barrier();

    // ---- what is left needs dZ only and runs side by side: wavefronts 0-3 take the loss, 4-7 the bias gradient, 8-15 the
    // tiles of dW; then all take tiles of dA ----
    // loss = (sum -t log(p + 1e-15)) / rows by 256 threads, partitioned and added as cce_fwd_kernel does.
    if (wave < 4) {
        double s = 0.0;
        if (p.loss != nullptr) {
            for (int e = tid; e < B * C; e += 256) {
                const int r = (int)(((float)e + 0.5f) * inv_C);
                s += (double)sT[r * L.CP + (e - r * C)];
            }
            s = wave_sum(s);
        }
        if (lane == 0) part[wave] = s;
    } else if (wave < 8) {
        // bias gradient = column sums of dZ by four wavefronts, every fourth row each, as colsum_block adds them (complete
        // groups of four of a wavefront's rows go to four accumulators in turn, what is left to the first); C <= 64
        if (p.dbias != nullptr) {
            const int j = lane, w = wave - 4;
            double acc0 = 0.0, acc1 = 0.0, acc2 = 0.0, acc3 = 0.0;
            if (j < C) {
                int i = w;
                for (; i + 12 < B; i += 16) {
                    const double a = (double)sD[i * L.CP + j], b = (double)sD[(i + 4) * L.CP + j];
                    const double c = (double)sD[(i + 8) * L.CP + j], d = (double)sD[(i + 12) * L.CP + j];
                    acc0 += a; acc1 += b; acc2 += c; acc3 += d;
                }
                for (; i < B; i += 4) acc0 += (double)sD[i * L.CP + j];
            }
            part[4 + w * 64 + lane] = (acc0 + acc1) + (acc2 + acc3);
        }
    } else if (p.dW != nullptr) {
        // dW = A^T . dZ
        const int tilesC = L.C16 / 16, tiles = tilesH * tilesC;
        for (int t = wave - 8; t < tiles; t += 8) {
            const int k0 = (t / tilesC) * 16, c0 = (t % tilesC) * 16;
            const Acc acc = chain(sA + g * L.HP + k0 + li, 4 * L.HP, sD + g * L.CP + c0 + li, 4 * L.CP, L.B16 / 4);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int k = k0 + MF::row(r, g), c = c0 + li;
                if (k < H && c < C) {
                    T* out = p.dW + k * C + c;
                    *out = p.accumulate_dW ? *out + acc[r] : acc[r];
                }
            }
        }
    }

    // ---- dA = dZ . W^T, times the derivative of the activation below ----
    if (p.dA != nullptr) {
        for (int first = wave; first < tiles_dA; first += HEAD_WAVES * DA_TILES) {
            if (first != wave) fetch_src(first);
#pragma unroll
            for (int q = 0; q < DA_TILES; ++q) {
                const int t = first + HEAD_WAVES * q;
                if (t >= tiles_dA) continue;
                const int i0 = (t / tilesH) * 16, k0 = (t % tilesH) * 16;
                const Acc acc = chain(sD + (i0 + li) * L.CP + g, 4, sW + (k0 + li) * L.CP + g, 4, L.C16 / 4);
                const int k = k0 + li;
                T* out = p.dA + (i0 + MF::row(0, g)) * H + k;
                const int row_step = (MF::row(1, g) - MF::row(0, g)) * H;
                if (p.act == ACT_LEAKYRELU || p.act == ACT_NONE) {  // (the common cases without the dispatch per element)
                    const T slope = p.act == ACT_NONE ? (T)1 : p.alpha;
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (i0 + MF::row(r, g) < B && k < H) out[r * row_step] = acc[r] * (src[q][r] > (T)0 || p.act == ACT_NONE ? (T)1 : slope);
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (i0 + MF::row(r, g) < B && k < H) out[r * row_step] = acc[r] * act_derivative<T>(p.act, src[q][r], p.alpha);
                }
            }
        }
    }
    lds_barrier();
    if (tid == 0 && p.loss != nullptr) p.loss[0] = (T)((part[0] + part[1]) + (part[2] + part[3])) / (T)B;
    if (wave == 1 && lane < C && p.dbias != nullptr)
        p.dbias[lane] = (T)((part[4 + lane] + part[4 + 64 + lane]) + (part[4 + 128 + lane] + part[4 + 192 + lane]));
}

}  // namespace

template <typename T>
size_t classifier_head_lds_bytes(int64_t B, int64_t H, int64_t C) {
    return HeadLayout<T>((int)B, (int)H, (int)C).bytes;
}

// Shapes the one-launch kernel takes: at most 64 classes, fewer than 2048 rows (the column sum of a taller batch is taken
// in chunks), everything within 144 KB of LDS (a batch of 64 rows of 128 inputs in double: 110 KB).
// PRAD_HEAD_FUSED=0 switches it off (a tuning aid).
template <typename T>
bool classifier_head_eligible(int64_t B, int64_t H, int64_t C) {
    static const bool enabled = [] { const char* e = getenv("PRAD_HEAD_FUSED"); return !(e && e[0] == '0'); }();
    if (!enabled || B < 1 || H < 1 || C < 1 || C > 64 || B >= COLSUM_CHUNK_ROWS || H > 8192) return false;
    return classifier_head_lds_bytes<T>(B, H, C) <= HEAD_MAX_LDS;
}

template <typename T>
hipError_t launch_classifier_head(const HeadArgs<T>& a, hipStream_t s) {
    if (!classifier_head_eligible<T>(a.B, a.H, a.C)) return hipErrorNotSupported;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(classifier_head_kernel<T>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)HEAD_MAX_LDS);
    if (attr != hipSuccess) return attr;
    hipLaunchKernelGGL((classifier_head_kernel<T>), dim3(1), dim3(HEAD_THREADS), classifier_head_lds_bytes<T>(a.B, a.H, a.C), s, a);
    return hipGetLastError();
}

#define INSTANTIATE(T)                                                       \
    template size_t classifier_head_lds_bytes<T>(int64_t, int64_t, int64_t);  \
    template bool classifier_head_eligible<T>(int64_t, int64_t, int64_t);     \
    template hipError_t launch_classifier_head<T>(const HeadArgs<T>&, hipStream_t);
INSTANTIATE(double)
INSTANTIATE(float)
#undef INSTANTIATE

}  // namespace prad
