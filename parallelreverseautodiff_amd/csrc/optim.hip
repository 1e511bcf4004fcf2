// GradientClipper.ClipGradients (src/RMAD/GradientClipper.cs:118-157 with StandardizedMatrix
// :212-253) and AdamOptimizer.UpdateWeightWithAdam (src/RMAD/AdamOptimizer.cs:195-239) as
// multi-tensor bandwidth kernels: one launch sequence covers every (weight, gradient, m, v)
// group of a model, replacing the Parallel.For over layers of GradientClipper.Clip (:31-71)
// and AdamOptimizer.Optimize (:32-91) and the five temporaries per weight of the reference.
//
// Work is cut into chunks of OPT_CHUNK elements; chunk c of the launch belongs to the tensor whose
// [first_chunk, first_chunk + nchunks) range contains it (binary search in the descriptor table).
//
// Clip statistics: the reference makes two passes (mean, then sum of squared deviations).  Here
// each chunk produces (count, mean, M2) with a shifted two-pass over its registers, chunks are
// merged with Chan's pairwise formula in double; this is as accurate as the two-pass form and
// reads the gradient once.  Then one pass clamps in place.  HBM traffic: 3 element sizes per
// element (read for statistics, read + write for the clamp).
#include "common.h"

#include <cstring>

namespace prad {

constexpr int OPT_THREADS = 256;
// Elements per workgroup (template argument CHUNK of the kernels): 4096, or for large float tensors 8192, so
// that a float workgroup keeps as many bytes in flight as a double one (float clip was 4 points of HBM peak
// behind with 4096-element chunks); a small model keeps the small chunk, which spreads it over more workgroups.
constexpr int OPT_CHUNK_SMALL = 4096;
template <typename T> constexpr int OPT_CHUNK_LARGE = 32768 / (int)sizeof(T);
constexpr int64_t LARGE_CHUNK_FROM = (int64_t)4 << 20;  // total elements of a launch
// Adam alone moves seven streams (four read, three written) per workgroup: there 16 KB per stream and workgroup is the
// better cut (64 Mi doubles: 0.69 to 0.705 of 8 TB/s with 32 KB, 0.72 to 0.74 with 16 KB or 8 KB; the arithmetic does
// not show in the time at all, and neither workgroups that loop over several chunks nor addresses of the four tensors
// skewed against each other gain anything).
template <typename T> constexpr int ADAM_CHUNK_LARGE = 16384 / (int)sizeof(T);
// A model of a few million parameters or less is only a few 4096-element chunks per compute unit, a small one not even
// one (the 235 000 of the 784-256-128-10 network: 58 workgroups, each moving its 229 KB at one compute unit's share of
// the bandwidth - 11 us for 13 MB); chunks of 1024 spread it over four times as many.
constexpr int OPT_CHUNK_TINY = 1024;
constexpr int64_t TINY_CHUNK_BELOW = (int64_t)4 << 20;  // total elements of a launch

template <typename T>
struct DevTensor {
    T* g; T* w; T* m; T* v;
    int64_t n;
    int64_t first_chunk;  // index of this tensor's first chunk in the launch
    int64_t nchunks;
};

constexpr int MAX_TABLE = 40;  // tensors per launch: the table travels as a kernel argument

template <typename T>
struct TensorTable {
    DevTensor<T> t[MAX_TABLE];
    int nt;
};

template <typename T>
__device__ __forceinline__ int find_tensor(const DevTensor<T>* t, int nt, int64_t chunk) {
    int lo = 0, hi = nt - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (t[mid].first_chunk <= chunk) lo = mid; else hi = mid - 1;
    }
    return lo;
}

struct Moments {
    double n, mean, m2;
};
__device__ __forceinline__ Moments merge(const Moments& a, const Moments& b) {
    if (b.n == 0.0) return a;
    if (a.n == 0.0) return b;
    Moments r;
    r.n = a.n + b.n;
    const double delta = b.mean - a.mean;
    r.mean = a.mean + delta * (b.n / r.n);
    r.m2 = a.m2 + b.m2 + delta * delta * (a.n * b.n / r.n);
    return r;
}
// Merge of two groups of equal size (no division): used inside full chunks, where every lane and
// every wavefront holds the same number of elements.
__device__ __forceinline__ Moments merge_equal(const Moments& a, const Moments& b) {
    Moments r;
    const double delta = b.mean - a.mean;
    r.n = a.n + a.n;
    r.mean = a.mean + 0.5 * delta;
    r.m2 = a.m2 + b.m2 + delta * delta * (0.5 * a.n);
    return r;
}
__device__ __forceinline__ Moments shfl_down(const Moments& a, int off) {
    Moments r;
    r.n = __shfl_down(a.n, off, 64);
    r.mean = __shfl_down(a.mean, off, 64);
    r.m2 = __shfl_down(a.m2, off, 64);
    return r;
}

// A chunk is processed with 16-byte vector accesses when it is full and its tensor's pointers are
// 16-byte aligned (chunks start at multiples of 32 KiB); partial last chunks and borrowed,
// unaligned buffers take the scalar path.
template <typename T> struct OptVec;
template <> struct OptVec<double> { typedef double type __attribute__((ext_vector_type(2))); static constexpr int N = 2; };
template <> struct OptVec<float> { typedef float type __attribute__((ext_vector_type(4))); static constexpr int N = 4; };

template <typename T, int CHUNK>
__device__ __forceinline__ bool vector_chunk(const void* a, const void* b, const void* c, const void* d, int64_t begin, int64_t end) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c) |
                           reinterpret_cast<uintptr_t>(d);
    return (end - begin == CHUNK) && (bits % 16 == 0);
}

// Per-chunk moments -> partial[chunk].
template <typename T, int CHUNK>
__global__ void __launch_bounds__(OPT_THREADS) clip_stats_kernel(const TensorTable<T> tab, Moments* __restrict__ partial) {
    typedef typename OptVec<T>::type V;
    constexpr int VN = OptVec<T>::N;
    const int64_t chunk = blockIdx.x;
    const int ti = find_tensor(tab.t, tab.nt, chunk);
    const DevTensor<T> t = tab.t[ti];
    const int64_t begin = (chunk - t.first_chunk) * CHUNK;
    const int64_t end = min(begin + (int64_t)CHUNK, t.n);
    constexpr int PER = CHUNK / OPT_THREADS;  // 4, 16 or 32 elements per thread
    double x[PER];
    int cnt = 0;
    double sum = 0.0;
    if (vector_chunk<T, CHUNK>(t.g, nullptr, nullptr, nullptr, begin, end)) {
        const V* __restrict__ gv = reinterpret_cast<const V*>(t.g + begin);
        V v[PER / VN];
#pragma unroll
        for (int e = 0; e < PER / VN; ++e) v[e] = __builtin_nontemporal_load(gv + e * OPT_THREADS + threadIdx.x);
#pragma unroll
        for (int e = 0; e < PER / VN; ++e)
#pragma unroll
            for (int c = 0; c < VN; ++c) { x[e * VN + c] = (double)v[e][c]; sum += x[e * VN + c]; }
        cnt = PER;
    } else {
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int64_t i = begin + (int64_t)e * OPT_THREADS + threadIdx.x;
            if (i < end) { x[e] = (double)t.g[i]; sum += x[e]; ++cnt; } else x[e] = 0.0;
        }
    }
    Moments mo;
    mo.n = (double)cnt;
    mo.mean = cnt > 0 ? sum / (double)cnt : 0.0;
    mo.m2 = 0.0;
    if (cnt == PER) {
#pragma unroll
        for (int e = 0; e < PER; ++e) { const double d = x[e] - mo.mean; mo.m2 += d * d; }
    } else {
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            const int64_t i = begin + (int64_t)e * OPT_THREADS + threadIdx.x;
            if (i < end) { const double d = x[e] - mo.mean; mo.m2 += d * d; }
        }
    }
    const bool full = end - begin == CHUNK;  // uniform over the workgroup
    if (full) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mo = merge_equal(mo, shfl_down(mo, off));
    } else {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mo = merge(mo, shfl_down(mo, off));
    }
    __shared__ Moments wave_part[OPT_THREADS / 64];
    if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = mo;
    __syncthreads();
    if (threadIdx.x == 0) {
        Moments r = wave_part[0];
        for (int w = 1; w < OPT_THREADS / 64; ++w) r = merge(r, wave_part[w]);
        partial[chunk] = r;
    }
}

// The whole workgroup merges the chunk moments [c0, c0 + nc) of one tensor; the result (mean,
// population standard deviation) is valid in thread 0.  Contains a barrier.
__device__ __forceinline__ void merge_tensor_chunks(const Moments* __restrict__ partial, int64_t c0, int64_t nc, double& mean,
                                                    double& stddev) {
    Moments mo{0.0, 0.0, 0.0};
    // Eight independent loads in flight per lane before the (serial) merges.
    for (int64_t c = threadIdx.x; c < nc; c += OPT_THREADS * 8) {
        Moments part[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int64_t idx = c + (int64_t)u * OPT_THREADS;
            part[u] = idx < nc ? partial[c0 + idx] : Moments{0.0, 0.0, 0.0};
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) mo = merge(mo, part[u]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mo = merge(mo, shfl_down(mo, off));
    __shared__ Moments wave_part[OPT_THREADS / 64];
    if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = mo;
    __syncthreads();
    mean = 0.0; stddev = 0.0;
    if (threadIdx.x == 0) {
        Moments r = wave_part[0];
        for (int w = 1; w < OPT_THREADS / 64; ++w) r = merge(r, wave_part[w]);
        mean = r.mean;
        stddev = sqrt(r.m2 / r.n);  // population standard deviation
    }
}

// One workgroup per tensor: stats[ti] = {mean, stddev}.
template <typename T>
__global__ void __launch_bounds__(OPT_THREADS) clip_finalize_kernel(const TensorTable<T> tab, const Moments* __restrict__ partial,
                                                                    double* __restrict__ stats) {
    const int ti = blockIdx.x;
    double mean, stddev;
    merge_tensor_chunks(partial, tab.t[ti].first_chunk, tab.t[ti].nchunks, mean, stddev);
    if (threadIdx.x == 0) {
        stats[2 * ti] = mean;
        stats[2 * ti + 1] = stddev;
    }
}

// Statistics of tensor ti for a workgroup of the clamping pass: read from stats when the finalize
// launch ran, otherwise (tensors of few chunks) merged here by every workgroup for itself, in the
// same order, which saves a launch where launches are what a step costs.
constexpr int64_t INLINE_FINALIZE_CHUNKS = 256;
template <typename T>
__device__ __forceinline__ void tensor_stats(const DevTensor<T>& t, int ti, const double* __restrict__ stats,
                                             const Moments* __restrict__ partial, T& mean, T& stddev) {
    if (stats != nullptr) {
        // PRADLite keeps mean and standard deviation in float.
        mean = (T)stats[2 * ti];
        stddev = (T)stats[2 * ti + 1];
        return;
    }
    __shared__ double sh[2];
    double m, sd;
    merge_tensor_chunks(partial, t.first_chunk, t.nchunks, m, sd);
    if (threadIdx.x == 0) { sh[0] = m; sh[1] = sd; }
    __syncthreads();
    mean = (T)sh[0];
    stddev = (T)sh[1];
}

// .NET Math.Min: NaN when either argument is NaN.
template <typename T>
__device__ __forceinline__ T dotnet_min(T a, T b) {
    if (a != a) return a;
    if (b != b) return b;
    return a < b ? a : b;
}

template <typename T>
struct Clamp {
    T mean, stddev, clip_value, min_value;
    __device__ __forceinline__ T operator()(T g) const {
        const T z = (g - mean) / stddev;
        const T value = dotnet_min<T>(clip_value, (T)1 + (z < (T)0 ? -z : z));
        if (g > value) g = value;
        else if (g < -value) g = -value;
        if (g > (T)0 && g < min_value) g = min_value;
        else if (g < (T)0 && g > -min_value) g = -min_value;
        return g;
    }
};

template <typename T>
struct AdamUpdate {
    T lr, beta1, beta2, omb1, omb2, c1, c2, eps;
    int reverse;  // 0: UpdateWeightWithAdam; 1: ReverseAdamUpdate (src/RMAD/AdamOptimizer.cs:158-193), statement for statement
    __device__ __forceinline__ void operator()(T& w, T& m, T& v, T g) const {
        if (reverse) {
            const T mhat = c1 * m;
            const T vhat = c2 * v;
            const T red = lr * mhat / (sqrt(vhat) + eps);
            w = w + red;
            m = (m - (omb1 * g)) / beta1;
            v = (v - ((omb2 * g) * g)) / beta2;
            return;
        }
        const T first = (beta1 * m) + (omb1 * g);
        const T second = (beta2 * v) + (omb2 * (g * g));
        const T mhat = c1 * first;
        const T vhat = c2 * second;
        const T red = lr * mhat / (sqrt(vhat) + eps);
        w = w - red;
        m = first;
        v = second;
    }
};

template <typename T, int CHUNK>
__global__ void __launch_bounds__(OPT_THREADS) clip_apply_kernel(const TensorTable<T> tab, const double* __restrict__ stats,
                                                                 const Moments* __restrict__ partial, T clip_value, T min_value) {
    const int64_t chunk = blockIdx.x;
    const int ti = find_tensor(tab.t, tab.nt, chunk);
    const DevTensor<T> t = tab.t[ti];
    Clamp<T> clamp;
    tensor_stats<T>(t, ti, stats, partial, clamp.mean, clamp.stddev);
    clamp.clip_value = clip_value; clamp.min_value = min_value;
    const int64_t begin = (chunk - t.first_chunk) * CHUNK;
    const int64_t end = min(begin + (int64_t)CHUNK, t.n);
    constexpr int PER = CHUNK / OPT_THREADS;
    if (vector_chunk<T, CHUNK>(t.g, nullptr, nullptr, nullptr, begin, end)) {
        typedef typename OptVec<T>::type V;
        constexpr int VN = OptVec<T>::N;
        V* __restrict__ gv = reinterpret_cast<V*>(t.g + begin);
        V v[PER / VN];
#pragma unroll
        for (int e = 0; e < PER / VN; ++e) v[e] = __builtin_nontemporal_load(gv + e * OPT_THREADS + threadIdx.x);
#pragma unroll
        for (int e = 0; e < PER / VN; ++e) {
#pragma unroll
            for (int c = 0; c < VN; ++c) v[e][c] = clamp(v[e][c]);
            __builtin_nontemporal_store(v[e], gv + e * OPT_THREADS + threadIdx.x);
        }
        return;
    }
#pragma unroll 4
    for (int e = 0; e < PER; ++e) {
        const int64_t i = begin + (int64_t)e * OPT_THREADS + threadIdx.x;
        if (i < end) t.g[i] = clamp(t.g[i]);
    }
}

// Adam: one pass over w, m, v, g (7 element sizes of HBM traffic per element).  With CLIP the clamping
// pass of the clipper runs in the same pass (the clamped gradient is stored, as the clipper does in
// place): 8 element sizes instead of 2 + 7 for the two passes.
template <typename T, int CHUNK, bool CLIP>
__global__ void __launch_bounds__(OPT_THREADS) adam_kernel(const TensorTable<T> tab, const AdamUpdate<T> update,
                                                           const double* __restrict__ stats, const Moments* __restrict__ partial,
                                                           T clip_value, T min_value) {
    const int64_t chunk = blockIdx.x;
    const int ti = find_tensor(tab.t, tab.nt, chunk);
    const DevTensor<T> t = tab.t[ti];
    Clamp<T> clamp{};
    if (CLIP) {
        tensor_stats<T>(t, ti, stats, partial, clamp.mean, clamp.stddev);
        clamp.clip_value = clip_value; clamp.min_value = min_value;
    }
    const int64_t begin = (chunk - t.first_chunk) * CHUNK;
    const int64_t end = min(begin + (int64_t)CHUNK, t.n);
    constexpr int PER = CHUNK / OPT_THREADS;
    if (vector_chunk<T, CHUNK>(t.w, t.m, t.v, t.g, begin, end)) {
        typedef typename OptVec<T>::type V;
        constexpr int VN = OptVec<T>::N;
        constexpr int NV = PER / VN;  // 16-byte vectors per thread and tensor
        V* __restrict__ wv = reinterpret_cast<V*>(t.w + begin);
        V* __restrict__ mv = reinterpret_cast<V*>(t.m + begin);
        V* __restrict__ vv = reinterpret_cast<V*>(t.v + begin);
        V* __restrict__ gv = reinterpret_cast<V*>(t.g + begin);
        // All loads of the chunk are issued before the first update: the arithmetic of a vector (a division and a
        // square root per element) then runs while the later vectors are still on their way, and the stores go out
        // as the updates finish.  Measured against two half-chunk passes: 68.0 -> 69.3 % of 8 TB/s in double,
        // 73.5 -> 74.5 % in float; plain instead of non-temporal loads or stores cost 4 to 6 points.
        V w[NV], m[NV], v[NV], g[NV];
#pragma unroll
        for (int e = 0; e < NV; ++e) {
            const int iv = e * OPT_THREADS + threadIdx.x;
            w[e] = __builtin_nontemporal_load(wv + iv);
            m[e] = __builtin_nontemporal_load(mv + iv);
            v[e] = __builtin_nontemporal_load(vv + iv);
            g[e] = __builtin_nontemporal_load(gv + iv);
        }
#pragma unroll
        for (int e = 0; e < NV; ++e) {
            const int iv = e * OPT_THREADS + threadIdx.x;
#pragma unroll
            for (int c = 0; c < VN; ++c) {
                T wi = w[e][c], mi = m[e][c], vi = v[e][c];
                if (CLIP) g[e][c] = clamp(g[e][c]);
                update(wi, mi, vi, g[e][c]);
                w[e][c] = wi; m[e][c] = mi; v[e][c] = vi;
            }
            if (CLIP) __builtin_nontemporal_store(g[e], gv + iv);
            __builtin_nontemporal_store(w[e], wv + iv);
            __builtin_nontemporal_store(m[e], mv + iv);
            __builtin_nontemporal_store(v[e], vv + iv);
        }
        return;
    }
#pragma unroll 4
    for (int e = 0; e < PER; ++e) {
        const int64_t i = begin + (int64_t)e * OPT_THREADS + threadIdx.x;
        if (i < end) {
            T wi = t.w[i], mi = t.m[i], vi = t.v[i], gi = t.g[i];
            if (CLIP) { gi = clamp(gi); t.g[i] = gi; }
            update(wi, mi, vi, gi);
            t.w[i] = wi; t.m[i] = mi; t.v[i] = vi;
        }
    }
}

template <typename T>
static int64_t build_table(const TensorDesc<T>* host, int nt, TensorTable<T>& tab, int CHUNK) {
    int64_t chunks = 0;
    tab.nt = nt;
    for (int i = 0; i < nt; ++i) {
        tab.t[i].g = host[i].g; tab.t[i].w = host[i].w; tab.t[i].m = host[i].m; tab.t[i].v = host[i].v;
        tab.t[i].n = host[i].n;
        tab.t[i].first_chunk = chunks;
        tab.t[i].nchunks = (host[i].n + CHUNK - 1) / CHUNK;
        chunks += tab.t[i].nchunks;
    }
    return chunks;
}

size_t clip_workspace_bytes(const int64_t* n, int nt) {
    // Groups of MAX_TABLE tensors run one after another on the stream and reuse the space.
    size_t worst = 0;
    for (int g0 = 0; g0 < nt; g0 += MAX_TABLE) {
        int64_t chunks = 0, total = 0;
        for (int i = g0; i < nt && i < g0 + MAX_TABLE; ++i) total += n[i];
        const int64_t chunk = total < TINY_CHUNK_BELOW ? OPT_CHUNK_TINY : OPT_CHUNK_SMALL;  // (of the two larger ones the smaller: an upper bound)
        for (int i = g0; i < nt && i < g0 + MAX_TABLE; ++i) chunks += (n[i] + chunk - 1) / chunk;
        const size_t need = (size_t)chunks * sizeof(Moments) + (size_t)MAX_TABLE * 16;
        if (need > worst) worst = need;
    }
    return worst + 64;
}

// One group of at most MAX_TABLE tensors: clip only (ADAM false), Adam only (CLIP false) or both in one pass.
template <typename T, int CHUNK, bool CLIP, bool ADAM>
static hipError_t launch_group(const TensorDesc<T>* host, int gn, void* workspace, T clip_value, T min_value,
                               const AdamUpdate<T>& update, hipStream_t s, const AdamLaunchObserver* obs) {
    TensorTable<T> tab;
    const int64_t chunks = build_table(host, gn, tab, CHUNK);
    if (chunks == 0) return hipSuccess;
    if (chunks > 0x7fffffffLL) return hipErrorInvalidValue;
    const double* stats = nullptr;
    const Moments* partial = nullptr;
    if (CLIP) {
        double* dstats = reinterpret_cast<double*>(workspace);
        Moments* dpartial = reinterpret_cast<Moments*>(static_cast<char*>(workspace) + (size_t)MAX_TABLE * 16);
        hipLaunchKernelGGL((clip_stats_kernel<T, CHUNK>), dim3((unsigned)chunks), dim3(OPT_THREADS), 0, s, tab, dpartial);
        int64_t most = 0;
        for (int i = 0; i < gn; ++i) most = tab.t[i].nchunks > most ? tab.t[i].nchunks : most;
        // Tensors of few chunks: the clamping pass merges the chunk moments itself and the finalize launch is skipped.
        if (most > INLINE_FINALIZE_CHUNKS) {
            hipLaunchKernelGGL((clip_finalize_kernel<T>), dim3((unsigned)gn), dim3(OPT_THREADS), 0, s, tab, dpartial, dstats);
            stats = dstats;
        }
        partial = dpartial;
    }
    if (ADAM) {
        hipLaunchKernelGGL((adam_kernel<T, CHUNK, CLIP>), dim3((unsigned)chunks), dim3(OPT_THREADS), 0, s, tab, update, stats, partial,
                           clip_value, min_value);
        if (obs != nullptr) obs->fn(obs->ctx, s);
    } else
        hipLaunchKernelGGL((clip_apply_kernel<T, CHUNK>), dim3((unsigned)chunks), dim3(OPT_THREADS), 0, s, tab, stats, partial,
                           clip_value, min_value);
    return hipGetLastError();
}

template <typename T, bool CLIP, bool ADAM>
static hipError_t launch_groups(const TensorDesc<T>* host, int nt, void* workspace, T clip_value, T min_value,
                                const AdamUpdate<T>& update, hipStream_t s, const AdamLaunchObserver* obs = nullptr) {
    for (int g0 = 0; g0 < nt; g0 += MAX_TABLE) {
        const int gn = nt - g0 < MAX_TABLE ? nt - g0 : MAX_TABLE;
        int64_t total = 0;
        for (int i = 0; i < gn; ++i) total += host[g0 + i].n;
        constexpr int LARGE = (ADAM && !CLIP) ? ADAM_CHUNK_LARGE<T> : OPT_CHUNK_LARGE<T>;
        const hipError_t e = total < TINY_CHUNK_BELOW
                                 ? launch_group<T, OPT_CHUNK_TINY, CLIP, ADAM>(host + g0, gn, workspace, clip_value, min_value, update, s, obs)
                             : (LARGE != OPT_CHUNK_SMALL && total >= LARGE_CHUNK_FROM)
                                 ? launch_group<T, LARGE, CLIP, ADAM>(host + g0, gn, workspace, clip_value, min_value, update, s, obs)
                                 : launch_group<T, OPT_CHUNK_SMALL, CLIP, ADAM>(host + g0, gn, workspace, clip_value, min_value, update, s, obs);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

template <typename T>
hipError_t launch_clip(const TensorDesc<T>* host, int nt, void* workspace, T clip_value, T min_value, hipStream_t s) {
    return launch_groups<T, true, false>(host, nt, workspace, clip_value, min_value, AdamUpdate<T>{}, s);
}

template <typename T>
hipError_t launch_adam(const TensorDesc<T>* host, int nt, T lr, T beta1, T beta2, T eps, T c1, T c2, bool reverse, hipStream_t s,
                       const AdamLaunchObserver* obs) {
    const AdamUpdate<T> update{lr, beta1, beta2, (T)1 - beta1, (T)1 - beta2, c1, c2, eps, reverse ? 1 : 0};
    return launch_groups<T, false, true>(host, nt, nullptr, (T)0, (T)0, update, s, obs);
}

// GradientClipper.Clip followed by AdamOptimizer.Optimize over the same tensors: statistics pass, then
// one pass that clamps the gradient and updates w, m, v.
template <typename T>
hipError_t launch_clip_adam(const TensorDesc<T>* host, int nt, void* workspace, T clip_value, T min_value, T lr, T beta1, T beta2,
                            T eps, T c1, T c2, hipStream_t s, const AdamLaunchObserver* obs) {
    const AdamUpdate<T> update{lr, beta1, beta2, (T)1 - beta1, (T)1 - beta2, c1, c2, eps, 0};
    return launch_groups<T, true, true>(host, nt, workspace, clip_value, min_value, update, s, obs);
}

// The bias-correction factors are launch arguments of the Adam kernel (argument 1, an AdamUpdate<T>).  A recorded
// launch sequence keeps the arguments it was recorded with; before a replay that stands for a later AdamIteration the
// factors of its Adam kernel nodes are replaced here, every other argument staying as recorded.
template <typename T>
hipError_t adam_node_set_bias_correction(hipGraphExec_t exec, hipGraphNode_t node, T c1, T c2) {
    hipKernelNodeParams kp;
    memset(&kp, 0, sizeof(kp));
    hipError_t e = hipGraphKernelNodeGetParams(node, &kp);
    if (e != hipSuccess) return e;
    if (kp.kernelParams == nullptr) return hipErrorInvalidValue;
    constexpr int NARGS = 6;  // tab, update, stats, partial, clip_value, min_value
    AdamUpdate<T> update = *static_cast<const AdamUpdate<T>*>(kp.kernelParams[1]);
    update.c1 = c1;
    update.c2 = c2;
    void* args[NARGS];
    for (int i = 0; i < NARGS; ++i) args[i] = kp.kernelParams[i];
    args[1] = &update;
    kp.kernelParams = args;
    kp.extra = nullptr;
    return hipGraphExecKernelNodeSetParams(exec, node, &kp);
}
template hipError_t adam_node_set_bias_correction<double>(hipGraphExec_t, hipGraphNode_t, double, double);
template hipError_t adam_node_set_bias_correction<float>(hipGraphExec_t, hipGraphNode_t, float, float);

template hipError_t launch_clip<double>(const TensorDesc<double>*, int, void*, double, double, hipStream_t);
template hipError_t launch_clip<float>(const TensorDesc<float>*, int, void*, float, float, hipStream_t);
template hipError_t launch_adam<double>(const TensorDesc<double>*, int, double, double, double, double, double, double, bool,
                                        hipStream_t, const AdamLaunchObserver*);
template hipError_t launch_adam<float>(const TensorDesc<float>*, int, float, float, float, float, float, float, bool, hipStream_t,
                                       const AdamLaunchObserver*);
template hipError_t launch_clip_adam<double>(const TensorDesc<double>*, int, void*, double, double, double, double, double, double,
                                             double, double, hipStream_t, const AdamLaunchObserver*);
template hipError_t launch_clip_adam<float>(const TensorDesc<float>*, int, void*, float, float, float, float, float, float, float,
                                            float, hipStream_t, const AdamLaunchObserver*);

}  // namespace prad
