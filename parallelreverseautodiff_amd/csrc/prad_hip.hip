// C ABI of libprad_hip.so (declared in include/prad_hip.h): lifecycle, device-resident matrices,
// and the entry points that enqueue the kernels of this library.  Replaces the per-call
// allocate / copy / launch / copy-back sequence of src/RMAD/GpuMatrixMultiplyOperation.cs:170-202
// and the serialise + thread-hop + cuBLAS path of src/RMAD/CudaBlas.cs:273-403.
//
// Threading model: one library stream; every entry point takes the context lock while it
// validates, (re)sizes shared staging/workspace and enqueues, so calls from any number of host
// threads are safe and execute in the order they acquired the lock.
#include "../../include/prad_hip.h"
#include "common.h"

#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <map>
#include <string>
#include <thread>
#include <vector>

using namespace prad;

struct prad_buf {
    uint32_t magic;
    int32_t dtype;
    int64_t depth, rows, cols;
    void* ptr;
    bool owned;
    size_t block_bytes;  // size class of the device block behind an owned buffer (0 for borrowed memory)
};

// Scratch of the allocation-free entry point (prad_clip_adam_multi_noalloc): device memory that exists from the
// moment the code object is loaded, one copy per GPU, held until the process ends.  In host code the name is only
// a stand-in for the symbol: its device address is asked for once per device (init_static_scratch) and every
// kernel argument uses that address.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)1 << 20;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

namespace {

constexpr uint32_t BUF_MAGIC = 0x50524144u;  // "PRAD"
constexpr size_t STAGING_CHUNK = (size_t)256 << 20;

constexpr size_t COUNTER_BYTES = 4096;  // arrival counters: one per tile of a split or paired product, and a few
constexpr size_t SEQ_FLAG_BYTES = 8192;  // two words per workgroup of an LSTM sequence kernel: progress, and where it runs
static_assert(COUNTER_BYTES >= GEMM_SPLIT_MAX_TILES * sizeof(unsigned), "a split product needs a counter per tile");

// One stream, one kernel workspace (partial results of split products, clip moments, loss partial sums, tall
// column sums) and one block of arrival counters: everything is enqueued in lock order, so no two kernels
// that use the workspace ever run side by side.
struct Context {
    std::mutex mu;
    std::atomic<bool> initialized{false};
    int device = -1;
    hipStream_t stream = nullptr;
    void* workspace = nullptr;
    size_t workspace_bytes = 0;
    std::vector<void*> retired_workspaces;  // outgrown blocks that recorded launch sequences may still address
    unsigned* counter = nullptr;            // zero between launches: the last workgroup to arrive resets its counter
    void* pinned = nullptr;
    size_t pinned_bytes = 0;
    // A launch sequence is being recorded by `recorder`; calls from other threads are refused meanwhile.
    bool recording = false;
    std::thread::id recorder;
    int live_graphs = 0;                    // recorded sequences not yet destroyed
    // LSTM sequence kernels: the workgroups' progress flags, and a word in host memory that a workgroup writes
    // when it gives up waiting for its peers (checked after every wait for the stream).
    unsigned* seq_flags = nullptr;
    unsigned* seq_abort = nullptr;          // hipHostMalloc'ed, also the address the kernels use
    int compute_units = 0;
    // Sequence kernels: off when PRAD_LSTM_SEQUENCE=0, when prad_lstm_sequence_enable(0) said so, when the co-residency
    // probe of a grid failed, or - sticky - once a sequence kernel gave up; seq_proven_grid is the largest grid
    // (workgroups) that a probe has shown the device to hold at once.
    bool seq_enabled = true;
    int seq_proven_grid = 0;
    bool seq_groups_local = false;          // the last probe found every row group on one XCD
    void* seq_step_scratch = nullptr;       // dh and dc ping-pong blocks of the per-time-step backward (kept: recordings address it)
    size_t seq_step_scratch_bytes = 0, seq_step_scratch_class = 0;
    // Device blocks that prad_buf_free handed back, by size class.  Everything the library enqueues runs on the one
    // stream in lock order, so a block may be handed out again at once: whatever still reads or writes it is ahead
    // in the stream of whatever the next owner enqueues.
    std::map<size_t, std::vector<void*>> pool;
    size_t pool_bytes = 0;
    size_t pool_limit = 0;                  // half of the device memory, or PRAD_POOL_MAX_BYTES
    bool poison_outputs = false;            // PRAD_POISON_OUTPUTS=1: unfilled outputs start as NaN bit patterns (a testing aid)
    int64_t stat_device_mallocs = 0, stat_device_frees = 0, stat_stream_syncs = 0, stat_pool_hits = 0;
};
Context g_ctx;
#define CUR_STREAM (g_ctx.stream)
#define CUR_WORKSPACE (g_ctx.workspace)
thread_local std::string tl_error;

int32_t fail(int32_t code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    tl_error = buf;
    return code;
}

// Every entry point that enqueues takes the context lock through this: while a thread records a launch sequence,
// calls from other threads are refused instead of being recorded into it.
#define ENQUEUE_LOCK()                                                                                \
    std::lock_guard<std::mutex> lock(g_ctx.mu);                                                       \
    do {                                                                                              \
        if (g_ctx.recording && g_ctx.recorder != std::this_thread::get_id())                          \
            return fail(PRAD_ERR_RECORDING, "another thread is recording a launch sequence; call again after its prad_graph_end"); \
    } while (0)
// For entry points that allocate, copy to or from the host, or wait for the device (lock held).
#define NOT_WHILE_RECORDING(what)                                                                     \
    do {                                                                                              \
        if (g_ctx.recording) return fail(PRAD_ERR_RECORDING, what " cannot be part of a recorded launch sequence"); \
    } while (0)

#define HIP_TRY(expr, code)                                                                           \
    do {                                                                                              \
        hipError_t e_ = (expr);                                                                       \
        if (e_ != hipSuccess) return fail((code), "%s failed: %s", #expr, hipGetErrorString(e_));     \
    } while (0)

#define REQUIRE_INIT()                                                                                \
    do {                                                                                              \
        if (!g_ctx.initialized.load()) return fail(PRAD_ERR_NOT_INITIALIZED, "prad_init has not been called"); \
        hipError_t e_ = hipSetDevice(g_ctx.device);                                                   \
        if (e_ != hipSuccess) return fail(PRAD_ERR_LAUNCH, "hipSetDevice failed: %s", hipGetErrorString(e_)); \
    } while (0)

inline bool valid(prad_buf_t b) { return b != nullptr && b->magic == BUF_MAGIC; }
inline size_t elem_size(int32_t dtype) { return dtype == PRAD_F64 ? 8 : 4; }
inline int64_t count(prad_buf_t b) { return b->depth * b->rows * b->cols; }

#define REQUIRE_BUF(b)                                                                                \
    do {                                                                                              \
        if (!valid(b)) return fail(PRAD_ERR_BAD_HANDLE, "%s is not a live buffer handle", #b);        \
    } while (0)

// Lock must be held.  Waits for everything enqueued on the library stream.
int32_t sync_all() {
    ++g_ctx.stat_stream_syncs;
    if (g_ctx.stream) HIP_TRY(hipStreamSynchronize(g_ctx.stream), PRAD_ERR_LAUNCH);
    if (g_ctx.seq_abort != nullptr && *static_cast<volatile unsigned*>(g_ctx.seq_abort) != 0u) {
        *static_cast<volatile unsigned*>(g_ctx.seq_abort) = 0u;
        g_ctx.seq_enabled = false;
        g_ctx.seq_proven_grid = 0;
        return fail(PRAD_ERR_LAUNCH, "an LSTM sequence kernel gave up waiting for its peer workgroups (the device did not run its whole "
                                     "grid at once); the buffers written since the last successful wait hold partial results.  The "
                                     "sequence kernels are now off: prad_lstm_sequence_fwd / _bwd run one launch per time step from here "
                                     "on (prad_lstm_sequence_enable(1) turns them back on)");
    }
    return PRAD_OK;
}
int32_t ensure_pinned(size_t bytes) {
    if (bytes <= g_ctx.pinned_bytes) return PRAD_OK;
    if (int32_t st = sync_all()) return st;
    if (g_ctx.pinned) (void)hipHostFree(g_ctx.pinned);
    g_ctx.pinned = nullptr;
    g_ctx.pinned_bytes = 0;
    HIP_TRY(hipHostMalloc(&g_ctx.pinned, bytes, hipHostMallocDefault), PRAD_ERR_ALLOC);
    g_ctx.pinned_bytes = bytes;
    return PRAD_OK;
}
void free_retired_workspaces() {
    for (void* p : g_ctx.retired_workspaces) (void)hipFree(p);
    g_ctx.retired_workspaces.clear();
}
// Grows the kernel workspace (lock held).  A recording cannot allocate: every shape is run once eagerly before it
// is recorded, and a call that would have to grow the workspace during a recording fails.  Recorded launch
// sequences keep the address of the workspace they were recorded with, so while any of them is alive an
// outgrown block is not freed but retired (it is released when the last sequence is destroyed, or at
// shutdown): a replay then still finds its own block, and replays and eager calls never run side by side.
int32_t ensure_workspace(size_t bytes) {
    if (bytes <= g_ctx.workspace_bytes) return PRAD_OK;
    if (g_ctx.recording)
        return fail(PRAD_ERR_RECORDING, "the workspace would have to grow during a recording: run the sequence once before recording it");
    bytes = (bytes + 4095) & ~(size_t)4095;
    void* fresh = nullptr;
    HIP_TRY(hipMalloc(&fresh, bytes), PRAD_ERR_ALLOC);
    if (g_ctx.workspace) {
        if (g_ctx.live_graphs > 0) {
            g_ctx.retired_workspaces.push_back(g_ctx.workspace);
        } else {
            if (int32_t st = sync_all()) { (void)hipFree(fresh); return st; }
            (void)hipFree(g_ctx.workspace);
        }
    }
    g_ctx.workspace = fresh;
    g_ctx.workspace_bytes = bytes;
    return PRAD_OK;
}

// ---- device blocks of the matrices -----------------------------------------------------------------------
// Size class of a block: quarter-octave steps (at most a quarter more than asked for), 256 bytes at least.
inline size_t size_class(size_t bytes) {
    if (bytes <= 256) return 256;
    const int top = 63 - __builtin_clzll((unsigned long long)(bytes - 1));  // bytes - 1 lies in [2^top, 2^(top+1))
    const size_t step = (size_t)1 << (top - 2);
    return (bytes + step - 1) & ~(step - 1);
}
// Lock held.  Gives every pooled block back to the device (after waiting for the stream: queued work may still use them).
int32_t pool_release_all() {
    if (g_ctx.pool_bytes == 0) return PRAD_OK;
    if (int32_t st = sync_all()) return st;
    for (auto& kv : g_ctx.pool)
        for (void* p : kv.second) { (void)hipFree(p); ++g_ctx.stat_device_frees; }
    g_ctx.pool.clear();
    g_ctx.pool_bytes = 0;
    return PRAD_OK;
}
// Lock held.  A block of at least `bytes`: one that prad_buf_free handed back if there is one of that class, else a
// fresh one (when the device is out of memory the pooled blocks are released and the allocation is tried again).
int32_t pool_take(size_t bytes, void** out, size_t* klass) {
    *klass = size_class(bytes);
    auto it = g_ctx.pool.find(*klass);
    if (it != g_ctx.pool.end() && !it->second.empty()) {
        *out = it->second.back();
        it->second.pop_back();
        g_ctx.pool_bytes -= *klass;
        ++g_ctx.stat_pool_hits;
        return PRAD_OK;
    }
    hipError_t e = hipMalloc(out, *klass);
    if (e == hipErrorOutOfMemory && g_ctx.pool_bytes > 0) {
        (void)hipGetLastError();
        if (int32_t st = pool_release_all()) return st;
        e = hipMalloc(out, *klass);
    }
    if (e != hipSuccess) return fail(PRAD_ERR_ALLOC, "hipMalloc of %zu bytes failed: %s", *klass, hipGetErrorString(e));
    ++g_ctx.stat_device_mallocs;
    return PRAD_OK;
}
// Lock held.  No wait and no hipFree: the block is kept for the next allocation of its class, unless the pool
// already holds its share of the device memory.
int32_t pool_give(void* p, size_t klass) {
    if (g_ctx.pool_bytes + klass > g_ctx.pool_limit) {
        if (int32_t st = sync_all()) return st;
        HIP_TRY(hipFree(p), PRAD_ERR_ALLOC);
        ++g_ctx.stat_device_frees;
        return PRAD_OK;
    }
    g_ctx.pool[klass].push_back(p);
    g_ctx.pool_bytes += klass;
    return PRAD_OK;
}

// ---- the static scratch of the allocation-free entry point ----------------------------------------------
constexpr int MAX_DEVICES = 64;
void* g_scratch_ptr[MAX_DEVICES] = {};  // device address of `scratch` on each GPU this process has initialised
// Lock held, `device` current.
int32_t init_static_scratch(int device) {
    if (device < 0 || device >= MAX_DEVICES) return fail(PRAD_ERR_ARG, "device %d beyond the %d this library keeps scratch for", device, MAX_DEVICES);
    if (g_scratch_ptr[device] != nullptr) return PRAD_OK;
    void* ptr = nullptr;
    HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), PRAD_ERR_NOT_INITIALIZED);
    if (ptr == nullptr) return fail(PRAD_ERR_NOT_INITIALIZED, "hipGetSymbolAddress returned no address for the static scratch");
    g_scratch_ptr[device] = ptr;
    return PRAD_OK;
}

// ---- recorded launch sequences ----------------------------------------------------------------------------
constexpr uint32_t GRAPH_MAGIC = 0x50524147u;  // "PRAG"
// An Adam kernel node of a recording: its bias-correction factors 1 / (1 - beta^t) are launch arguments, so every
// replay that stands for a later AdamIteration gets them replaced (the reference's caller advances AdamIteration
// once per step, src/RMAD/AdamOptimizer.cs:204-207).
struct AdamNode {
    hipGraphNode_t node;
    int32_t dtype;
    double beta1, beta2;
    double t;        // AdamIteration the node was recorded with
    double applied;  // AdamIteration its current arguments stand for
};
struct RecordedGraph {
    uint32_t magic;
    hipGraph_t graph;
    hipGraphExec_t exec;
    std::vector<AdamNode> adam;
    double base_t;  // smallest recorded AdamIteration
    double next_t;  // AdamIteration the next launch gives the nodes recorded with base_t
};
constexpr int MAX_ADAM_NODES = 64;
AdamNode g_recording_adam[MAX_ADAM_NODES];  // nodes of the open recording (lock held whenever touched)
int g_recording_adam_count = 0;
bool g_recording_failed = false;

struct PendingAdam { int32_t dtype; double beta1, beta2, t; };
void note_adam_node(void* ctx, hipStream_t s) {
    const PendingAdam* pa = static_cast<const PendingAdam*>(ctx);
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long id = 0;
    hipGraph_t graph = nullptr;
    const hipGraphNode_t* deps = nullptr;
    size_t ndeps = 0;
    if (hipStreamGetCaptureInfo_v2(s, &status, &id, &graph, &deps, &ndeps) != hipSuccess || status != hipStreamCaptureStatusActive ||
        ndeps != 1 || g_recording_adam_count >= MAX_ADAM_NODES) {
        g_recording_failed = true;  // reported by prad_graph_end
        return;
    }
    g_recording_adam[g_recording_adam_count++] = AdamNode{deps[0], pa->dtype, pa->beta1, pa->beta2, pa->t, pa->t};
}

// 1 / (1 - Math.Pow(beta, AdamIteration)), src/RMAD/AdamOptimizer.cs:204-207; PRADLite: every parameter is a float and
// PradMath.Pow(float, float) is (float)Math.Pow.
inline void bias_correction(double beta1, double beta2, double t, double* c1, double* c2) {
    *c1 = 1 / (1 - std::pow(beta1, t));
    *c2 = 1 / (1 - std::pow(beta2, t));
}
inline void bias_correction(float b1, float b2, float tf, float* c1, float* c2) {
    *c1 = 1 / (1 - (float)std::pow((double)b1, (double)tf));
    *c2 = 1 / (1 - (float)std::pow((double)b2, (double)tf));
}

int32_t same_dtype(std::initializer_list<prad_buf_t> bufs) {
    int32_t dt = -1;
    for (prad_buf_t b : bufs) {
        if (b == nullptr) continue;
        if (dt < 0) dt = b->dtype;
        else if (b->dtype != dt) return fail(PRAD_ERR_DTYPE, "buffers of different element types in one call");
    }
    return PRAD_OK;
}

template <typename T>
GemmArgs<T> plain_gemm(int transA, int transB, int64_t M, int64_t N, int64_t K, const void* A, int64_t lda, const void* B,
                       int64_t ldb, void* C, int64_t ldc, int accumulate) {
    GemmArgs<T> a{};
    a.transA = transA; a.transB = transB;
    a.M = M; a.N = N; a.K = K;
    a.A = static_cast<const T*>(A); a.lda = lda;
    a.B = static_cast<const T*>(B); a.ldb = ldb;
    a.C = static_cast<T*>(C); a.ldc = ldc;
    a.accumulate = accumulate;
    a.batch = 1;
    return a;
}

// Products split along K (in several passes, or as pairs of workgroups per tile) need room for their
// partial results; the workspace is grown here (lock held).
template <typename T>
int32_t attach_split_workspace(GemmArgs<T>& a) {
    if constexpr (sizeof(T) == 4) {
        if (const size_t bytes = gemm_skinny_workspace_bytes(a)) {  // one pass over both operands, partial outputs per workgroup
            if (int32_t st = ensure_workspace(bytes)) return st;
            a.split_ws = static_cast<T*>(CUR_WORKSPACE);
            a.split_counters = g_ctx.counter;
            return PRAD_OK;
        }
    }
    // (in launch_gemm's order: split along K, else tiles shared several ways, else pairs of workgroups - a product that
    // qualifies for the last two is launched on shared tiles and needs their room)
    const int splits = gemm_split_factor(a.M, a.N, a.K, a.batch, (int)sizeof(T));
    int shared_tiles = 0;
    const int shared = splits <= 1 ? gemm_shared_tiles_plan(a.M, a.N, a.K, a.batch, (int)sizeof(T), &shared_tiles) : 0;
    const bool pairs = splits <= 1 && shared <= 1 && gemm_pairs(a.M, a.N, a.K, a.batch, (int)sizeof(T));
    if (splits <= 1 && !pairs && shared <= 1) return PRAD_OK;
    const size_t bytes = shared > 1 ? (size_t)shared_tiles * shared * 128 * 128 * sizeof(T)
                                  : (size_t)(pairs ? 2 : splits) * a.batch * a.M * a.N * sizeof(T);
    if (int32_t st = ensure_workspace(bytes)) return st;
    a.split_ws = static_cast<T*>(CUR_WORKSPACE);
    a.split_counters = g_ctx.counter;
    return PRAD_OK;
}

// Rows/columns of op(X) for a 2-D (per-slice) buffer.
inline int64_t op_rows(prad_buf_t b, int trans) { return trans ? b->cols : b->rows; }
inline int64_t op_cols(prad_buf_t b, int trans) { return trans ? b->rows : b->cols; }

struct Epilogue {
    prad_buf_t bias = nullptr;
    prad_buf_t Z = nullptr;
    int act_fwd = PRAD_ACT_NONE;
    int act_bwd = PRAD_ACT_NONE;
    prad_buf_t act_src = nullptr;
    double alpha = 0.0;
    // column sum riding along with the launch: colsum_dst (1 x cols) = column sums of colsum_src
    prad_buf_t colsum_src = nullptr;
    prad_buf_t colsum_dst = nullptr;
};

template <typename T>
GemmArgs<T> gemm_args_of(int transA, int transB, prad_buf_t A, prad_buf_t B, prad_buf_t C, int accumulate, const Epilogue& ep,
                         bool batched) {
    const int64_t M = op_rows(A, transA), K = op_cols(A, transA), N = op_cols(B, transB);
    GemmArgs<T> a = plain_gemm<T>(transA, transB, M, N, K, A->ptr, A->cols, B->ptr, B->cols, C->ptr, C->cols, accumulate);
    if (ep.bias) a.bias = static_cast<const T*>(ep.bias->ptr);
    if (ep.Z) { a.Z = static_cast<T*>(ep.Z->ptr); a.ldz = ep.Z->cols; }
    a.act_fwd = ep.act_fwd;
    a.act_bwd = ep.act_bwd;
    if (ep.act_src) { a.act_src = static_cast<const T*>(ep.act_src->ptr); a.ld_act = ep.act_src->cols; }
    a.alpha = (T)ep.alpha;
    if (ep.colsum_dst) {
        a.colsum_src = static_cast<const T*>(ep.colsum_src->ptr);
        a.colsum_dst = static_cast<T*>(ep.colsum_dst->ptr);
        a.colsum_rows = ep.colsum_src->rows;
        a.colsum_cols = ep.colsum_src->cols;
    }
    if (batched) {
        a.batch = (int)C->depth;
        a.strideA = A->depth == 1 ? 0 : A->rows * A->cols;
        a.strideB = B->depth == 1 ? 0 : B->rows * B->cols;
        a.strideC = C->rows * C->cols;
    }
    return a;
}

template <typename T>
int32_t enqueue_gemm_t(int transA, int transB, prad_buf_t A, prad_buf_t B, prad_buf_t C, int accumulate, const Epilogue& ep,
                       bool batched) {
    GemmArgs<T> a = gemm_args_of<T>(transA, transB, A, B, C, accumulate, ep, batched);
    if (int32_t st = attach_split_workspace(a)) return st;
    HIP_TRY(launch_gemm<T>(a, CUR_STREAM), PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

// Checks the operands of C = op(A).op(B) and of its epilogue, with the reference's messages.
int32_t validate_gemm(int transA, int transB, prad_buf_t A, prad_buf_t B, prad_buf_t C, const Epilogue& ep, bool batched) {
    REQUIRE_BUF(A); REQUIRE_BUF(B); REQUIRE_BUF(C);
    if ((transA != 0 && transA != 1) || (transB != 0 && transB != 1) || (transA && transB))
        return fail(PRAD_ERR_ARG, "unsupported transpose combination (%d, %d)", transA, transB);
    if (int32_t st = same_dtype({A, B, C, ep.bias, ep.Z, ep.act_src, ep.colsum_src, ep.colsum_dst})) return st;
    if (op_cols(A, transA) != op_rows(B, transB))
        return fail(PRAD_ERR_SHAPE, "Input 1 columns do not match Input 2 rows");
    if (C->rows != op_rows(A, transA) || C->cols != op_cols(B, transB))
        return fail(PRAD_ERR_ARG, "Cannot multiply %lldx%lld matrix by %lldx%lld matrix into %lldx%lld",
                    (long long)op_rows(A, transA), (long long)op_cols(A, transA), (long long)op_rows(B, transB),
                    (long long)op_cols(B, transB), (long long)C->rows, (long long)C->cols);
    if (batched) {
        if ((A->depth != 1 && A->depth != C->depth) || (B->depth != 1 && B->depth != C->depth))
            return fail(PRAD_ERR_SHAPE, "batched product: operand depth must be 1 or equal to the output depth");
    } else if (A->depth != 1 || B->depth != 1 || C->depth != 1) {
        return fail(PRAD_ERR_SHAPE, "deep buffer passed to a single product; use prad_gemm_batched");
    }
    if (ep.bias && (ep.bias->rows != 1 || ep.bias->cols != C->cols || ep.bias->depth != 1))
        return fail(PRAD_ERR_ARG, "The length of the bias vector must be the same as the number of columns in the input matrix.");
    if (ep.Z && (ep.Z->rows != C->rows || ep.Z->cols != C->cols || ep.Z->depth != C->depth))
        return fail(PRAD_ERR_ARG, "pre-activation buffer must have the shape of the output");
    if (ep.act_bwd != PRAD_ACT_NONE) {
        if (!valid(ep.act_src)) return fail(PRAD_ERR_BAD_HANDLE, "act_src is not a live buffer handle");
        if (ep.act_src->rows != C->rows || ep.act_src->cols != C->cols || ep.act_src->depth != C->depth)
            return fail(PRAD_ERR_ARG, "act_src must have the shape of the gradient it scales");
    }
    if (ep.act_fwd < 0 || ep.act_fwd > PRAD_ACT_AMPLIFIED_SIGMOID || ep.act_bwd < 0 || ep.act_bwd > PRAD_ACT_AMPLIFIED_SIGMOID)
        return fail(PRAD_ERR_ARG, "unknown activation selector");
    return PRAD_OK;
}

// Validates and enqueues C = op(A).op(B).
int32_t enqueue_gemm(int transA, int transB, prad_buf_t A, prad_buf_t B, prad_buf_t C, int accumulate, const Epilogue& ep,
                     bool batched) {
    if (int32_t st = validate_gemm(transA, transB, A, B, C, ep, batched)) return st;
    if (A->dtype == PRAD_F64) return enqueue_gemm_t<double>(transA, transB, A, B, C, accumulate, ep, batched);
    return enqueue_gemm_t<float>(transA, transB, A, B, C, accumulate, ep, batched);
}

// dA = dC . B^T (epilogue ep) and dB = A^T . dC (epilogue rider) in one launch where launch_gemm_pair takes them;
// *done says whether it did.  Operands already validated.
template <typename T>
int32_t enqueue_gradient_pair_t(prad_buf_t dC, prad_buf_t A, prad_buf_t B, prad_buf_t dA, prad_buf_t dB, int acc_dA, int acc_dB,
                                const Epilogue& ep, const Epilogue& rider, bool* done) {
    const GemmArgs<T> first = gemm_args_of<T>(0, 1, dC, B, dA, acc_dA, ep, false);
    const GemmArgs<T> second = gemm_args_of<T>(1, 0, A, dC, dB, acc_dB, rider, false);
    const hipError_t e = launch_gemm_pair<T>(first, second, CUR_STREAM);
    *done = e == hipSuccess;
    if (e != hipSuccess && e != hipErrorNotSupported) HIP_TRY(e, PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

// C = sum_q A[q].B[q] + bias: the pairs are the splits of one product along the joint reduction.
template <typename T>
int32_t batch_sum_fwd_t(prad_buf_t A, prad_buf_t B, prad_buf_t bias, prad_buf_t C) {
    GemmArgs<T> a = plain_gemm<T>(0, 0, A->rows, B->cols, A->cols, A->ptr, A->cols, B->ptr, B->cols, C->ptr, C->cols, 0);
    if (bias) a.bias = static_cast<const T*>(bias->ptr);
    if (A->depth > 1) {
        a.nseg = (int)A->depth;
        a.segstrideA = A->rows * A->cols;
        a.segstrideB = B->rows * B->cols;
        if (int32_t st = ensure_workspace((size_t)a.nseg * a.M * a.N * sizeof(T))) return st;
        a.split_ws = static_cast<T*>(CUR_WORKSPACE);
    } else if (int32_t st = attach_split_workspace(a)) {
        return st;
    }
    HIP_TRY(launch_gemm<T>(a, CUR_STREAM), PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

// One LSTM time step in one launch each way; shapes the fused kernels do not take run as product + cell kernel.
template <typename T>
int32_t lstm_step_fwd_t(prad_buf_t h_prev, prad_buf_t Wh, prad_buf_t G, prad_buf_t c_prev, prad_buf_t c, prad_buf_t tanh_c,
                        prad_buf_t h) {
    const int64_t rows = c->rows, H = c->cols;
    GemmArgs<T> a = plain_gemm<T>(0, 0, rows, 4 * H, H, h_prev->ptr, H, Wh->ptr, 4 * H, G->ptr, 4 * H, 1);
    a.lstm_hidden = H;
    a.lstm_c_prev = static_cast<const T*>(c_prev->ptr);
    a.lstm_c = static_cast<T*>(c->ptr); a.lstm_tanh_c = static_cast<T*>(tanh_c->ptr); a.lstm_h = static_cast<T*>(h->ptr);
    hipError_t e = launch_lstm_step_fwd<T>(a, CUR_STREAM);
    if (e == hipErrorNotSupported) {
        if (int32_t st = attach_split_workspace(a)) return st;
        HIP_TRY(launch_gemm<T>(a, CUR_STREAM), PRAD_ERR_LAUNCH);
        e = launch_lstm_cell_fwd<T>(static_cast<T*>(G->ptr), a.lstm_c_prev, a.lstm_c, a.lstm_tanh_c, a.lstm_h, rows, H, CUR_STREAM);
    }
    HIP_TRY(e, PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

template <typename T>
int32_t lstm_step_bwd_t(prad_buf_t dG_next, prad_buf_t Wh, prad_buf_t gates, prad_buf_t c_prev, prad_buf_t tanh_c,
                        prad_buf_t dh_loss, prad_buf_t dc_in, prad_buf_t dG, prad_buf_t dc_prev, prad_buf_t dh_scratch) {
    const int64_t rows = c_prev->rows, H = c_prev->cols;
    GemmArgs<T> a = plain_gemm<T>(0, 1, rows, H, 4 * H, dG_next->ptr, 4 * H, Wh->ptr, 4 * H, dh_scratch->ptr, H, 0);
    if (int32_t st = attach_split_workspace(a)) return st;
    a.lstm_hidden = H;
    a.lstm_gates = static_cast<const T*>(gates->ptr); a.lstm_c_prev = static_cast<const T*>(c_prev->ptr);
    a.lstm_tanh_c_in = static_cast<const T*>(tanh_c->ptr); a.lstm_dh_loss = static_cast<const T*>(dh_loss->ptr);
    a.lstm_dc_in = dc_in ? static_cast<const T*>(dc_in->ptr) : nullptr;
    a.lstm_dG = static_cast<T*>(dG->ptr); a.lstm_dc_prev = static_cast<T*>(dc_prev->ptr);
    hipError_t e = launch_lstm_step_bwd<T>(a, CUR_STREAM);
    if (e == hipErrorNotSupported) {
        HIP_TRY(launch_gemm<T>(a, CUR_STREAM), PRAD_ERR_LAUNCH);  // dh_scratch = dG_next . Wh^T
        e = launch_lstm_cell_bwd<T>(a.lstm_gates, a.lstm_c_prev, a.lstm_tanh_c_in, a.lstm_dh_loss, static_cast<const T*>(dh_scratch->ptr),
                                    a.lstm_dc_in, a.lstm_dG, a.lstm_dc_prev, rows, H, CUR_STREAM);
    }
    HIP_TRY(e, PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

int32_t same_shape(prad_buf_t a, prad_buf_t b, const char* what) {
    if (a->depth != b->depth || a->rows != b->rows || a->cols != b->cols)
        return fail(PRAD_ERR_ARG, "%s: Matrices must have the same dimensions.", what);
    return PRAD_OK;
}

}  // namespace

#pragma GCC visibility push(default)
extern "C" {

// ---------------------------------------------------------------------------------------------
int32_t prad_init(int32_t device_id) {
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    if (g_ctx.initialized.load()) {
        if (device_id == g_ctx.device) return PRAD_OK;
        return fail(PRAD_ERR_ARG, "already initialized on device %d", g_ctx.device);
    }
    int ndev = 0;
    HIP_TRY(hipGetDeviceCount(&ndev), PRAD_ERR_NOT_INITIALIZED);
    if (device_id < 0 || device_id >= ndev) return fail(PRAD_ERR_ARG, "device %d out of range (%d devices)", device_id, ndev);
    HIP_TRY(hipSetDevice(device_id), PRAD_ERR_NOT_INITIALIZED);
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device_id), PRAD_ERR_NOT_INITIALIZED);
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(PRAD_ERR_NOT_INITIALIZED, "device %d is %s; this library is built for gfx950 only", device_id, prop.gcnArchName);
    HIP_TRY(hipStreamCreateWithFlags(&g_ctx.stream, hipStreamNonBlocking), PRAD_ERR_NOT_INITIALIZED);
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&g_ctx.counter), COUNTER_BYTES), PRAD_ERR_ALLOC);
    HIP_TRY(hipMemset(g_ctx.counter, 0, COUNTER_BYTES), PRAD_ERR_ALLOC);
    if (int32_t st = init_static_scratch(device_id)) return st;
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&g_ctx.seq_flags), SEQ_FLAG_BYTES), PRAD_ERR_ALLOC);
    HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&g_ctx.seq_abort), 64, hipHostMallocDefault), PRAD_ERR_ALLOC);
    g_ctx.seq_abort[0] = 0u; g_ctx.seq_abort[1] = 0u;
    g_ctx.compute_units = std::min<int>(prop.multiProcessorCount, (int)(SEQ_FLAG_BYTES / (2 * sizeof(unsigned))));
    {
        const char* e = getenv("PRAD_LSTM_SEQUENCE");
        g_ctx.seq_enabled = !(e && e[0] == '0');
        g_ctx.seq_proven_grid = 0;
    }
    g_ctx.pool_limit = prop.totalGlobalMem / 2;
    if (const char* cap = getenv("PRAD_POOL_MAX_BYTES")) g_ctx.pool_limit = (size_t)strtoull(cap, nullptr, 10);
    if (const char* poison = getenv("PRAD_POISON_OUTPUTS")) g_ctx.poison_outputs = poison[0] == '1';
    g_ctx.recording = false;
    g_ctx.live_graphs = 0;
    g_ctx.device = device_id;
    g_ctx.initialized.store(true);
    return PRAD_OK;
}

int32_t prad_shutdown(void) {
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    if (!g_ctx.initialized.load()) return PRAD_OK;
    (void)hipSetDevice(g_ctx.device);
    (void)sync_all();
    if (g_ctx.seq_step_scratch) (void)pool_give(g_ctx.seq_step_scratch, g_ctx.seq_step_scratch_class);
    g_ctx.seq_step_scratch = nullptr; g_ctx.seq_step_scratch_bytes = 0;

    (void)pool_release_all();
    if (g_ctx.pinned) (void)hipHostFree(g_ctx.pinned);
    if (g_ctx.workspace) (void)hipFree(g_ctx.workspace);
    free_retired_workspaces();
    if (g_ctx.counter) (void)hipFree(g_ctx.counter);
    if (g_ctx.seq_flags) (void)hipFree(g_ctx.seq_flags);
    if (g_ctx.seq_abort) (void)hipHostFree(g_ctx.seq_abort);
    g_ctx.seq_flags = nullptr; g_ctx.seq_abort = nullptr;
    if (g_ctx.stream) (void)hipStreamDestroy(g_ctx.stream);
    g_ctx.workspace = nullptr; g_ctx.workspace_bytes = 0;
    g_ctx.counter = nullptr;
    g_ctx.pinned = nullptr; g_ctx.pinned_bytes = 0;
    g_ctx.stream = nullptr;
    g_ctx.recording = false;
    g_ctx.live_graphs = 0;
    g_ctx.device = -1;
    g_ctx.initialized.store(false);
    return PRAD_OK;
}

int32_t prad_is_initialized(void) { return g_ctx.initialized.load() ? 1 : 0; }
int32_t prad_device_id(void) { return g_ctx.device; }
const char* prad_last_error(void) { return tl_error.c_str(); }
void* prad_stream(void) { return g_ctx.stream; }

int32_t prad_stream_sync(void) {
    REQUIRE_INIT();
    ENQUEUE_LOCK();
    NOT_WHILE_RECORDING("waiting for the device");
    return sync_all();
}

// ---------------------------------------------------------------------------------------------
// Lock taken here.  zero_fill: new Matrix(rows, cols) starts at zero (src/RMAD/Matrix.cs:43-55); an output that the
// next kernel overwrites whole needs no fill launch.
static int32_t buf_alloc(int32_t dtype, int64_t depth, int64_t rows, int64_t cols, bool zero_fill, prad_buf_t* out) {
    REQUIRE_INIT();
    if (out == nullptr) return fail(PRAD_ERR_ARG, "out is NULL");
    *out = nullptr;
    if (dtype != PRAD_F64 && dtype != PRAD_F32) return fail(PRAD_ERR_DTYPE, "unknown dtype %d", dtype);
    if (depth <= 0 || rows <= 0 || cols <= 0) return fail(PRAD_ERR_ARG, "matrix dimensions must be positive");
    const size_t bytes = (size_t)depth * rows * cols * elem_size(dtype);
    void* p = nullptr;
    size_t klass = 0;
    ENQUEUE_LOCK();
    NOT_WHILE_RECORDING("an allocation");
    if (int32_t st = pool_take(bytes, &p, &klass)) return st;
    if (zero_fill) {
        hipError_t e = dtype == PRAD_F64 ? launch_fill_zero<double>(static_cast<double*>(p), depth * rows * cols, CUR_STREAM)
                                         : launch_fill_zero<float>(static_cast<float*>(p), depth * rows * cols, CUR_STREAM);
        if (e != hipSuccess) { (void)pool_give(p, klass); return fail(PRAD_ERR_LAUNCH, "zero fill failed: %s", hipGetErrorString(e)); }
    } else if (g_ctx.poison_outputs) {
        // every byte 0xFF is a NaN in both element types: an output that its kernel does not write whole shows up in any comparison
        if (hipMemsetAsync(p, 0xFF, bytes, CUR_STREAM) != hipSuccess) { (void)pool_give(p, klass); return fail(PRAD_ERR_LAUNCH, "poison fill failed"); }
    }
    *out = new prad_buf{BUF_MAGIC, dtype, depth, rows, cols, p, true, klass};
    return PRAD_OK;
}

int32_t prad_buf_alloc_deep(int32_t dtype, int64_t depth, int64_t rows, int64_t cols, prad_buf_t* out) {
    return buf_alloc(dtype, depth, rows, cols, true, out);
}

int32_t prad_buf_alloc(int32_t dtype, int64_t rows, int64_t cols, prad_buf_t* out) {
    return buf_alloc(dtype, 1, rows, cols, true, out);
}

int32_t prad_buf_alloc_output(int32_t dtype, int64_t depth, int64_t rows, int64_t cols, prad_buf_t* out) {
    return buf_alloc(dtype, depth, rows, cols, false, out);
}

int32_t prad_pool_trim(void) {
    REQUIRE_INIT();
    ENQUEUE_LOCK();
    NOT_WHILE_RECORDING("releasing pooled device memory");
    return pool_release_all();
}

int32_t prad_alloc_stats(int64_t* device_mallocs, int64_t* device_frees, int64_t* stream_syncs, int64_t* pool_hits,
                         int64_t* pooled_bytes) {
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    if (device_mallocs) *device_mallocs = g_ctx.stat_device_mallocs;
    if (device_frees) *device_frees = g_ctx.stat_device_frees;
    if (stream_syncs) *stream_syncs = g_ctx.stat_stream_syncs;
    if (pool_hits) *pool_hits = g_ctx.stat_pool_hits;
    if (pooled_bytes) *pooled_bytes = (int64_t)g_ctx.pool_bytes;
    return PRAD_OK;
}

int32_t prad_buf_wrap_deep(int32_t dtype, int64_t depth, int64_t rows, int64_t cols, void* device_ptr, prad_buf_t* out) {
    REQUIRE_INIT();
    if (out == nullptr || device_ptr == nullptr) return fail(PRAD_ERR_ARG, "NULL argument");
    if (dtype != PRAD_F64 && dtype != PRAD_F32) return fail(PRAD_ERR_DTYPE, "unknown dtype %d", dtype);
    if (depth <= 0 || rows <= 0 || cols <= 0) return fail(PRAD_ERR_ARG, "matrix dimensions must be positive");
    *out = new prad_buf{BUF_MAGIC, dtype, depth, rows, cols, device_ptr, false, 0};
    return PRAD_OK;
}

int32_t prad_buf_wrap(int32_t dtype, int64_t rows, int64_t cols, void* device_ptr, prad_buf_t* out) {
    return prad_buf_wrap_deep(dtype, 1, rows, cols, device_ptr, out);
}

int32_t prad_buf_free(prad_buf_t b) {
    if (b == nullptr) return PRAD_OK;
    REQUIRE_BUF(b);
    if (b->owned) {
        REQUIRE_INIT();
        ENQUEUE_LOCK();
        NOT_WHILE_RECORDING("freeing a buffer");
        // Work that still uses the buffer may be queued: the block goes back to the pool, and whoever gets it next
        // enqueues behind that work.
        if (int32_t st = pool_give(b->ptr, b->block_bytes)) return st;
    }
    b->magic = 0;
    delete b;
    return PRAD_OK;
}

int32_t prad_buf_shape(prad_buf_t b, int64_t* depth, int64_t* rows, int64_t* cols, int32_t* dtype) {
    REQUIRE_BUF(b);
    if (depth) *depth = b->depth;
    if (rows) *rows = b->rows;
    if (cols) *cols = b->cols;
    if (dtype) *dtype = b->dtype;
    return PRAD_OK;
}

void* prad_buf_device_ptr(prad_buf_t b) { return valid(b) ? b->ptr : nullptr; }

int32_t prad_buf_zero(prad_buf_t b) {
    REQUIRE_INIT();
    REQUIRE_BUF(b);
    ENQUEUE_LOCK();
    if (b->dtype == PRAD_F64) HIP_TRY(launch_fill_zero<double>(static_cast<double*>(b->ptr), count(b), CUR_STREAM), PRAD_ERR_LAUNCH);
    else HIP_TRY(launch_fill_zero<float>(static_cast<float*>(b->ptr), count(b), CUR_STREAM), PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

int32_t prad_zero_multi(const prad_buf_t* bufs, int32_t n) {
    REQUIRE_INIT();
    if (n < 0 || (n > 0 && bufs == nullptr)) return fail(PRAD_ERR_ARG, "bad tensor list");
    std::vector<void*> ptrs;
    std::vector<size_t> bytes;
    std::vector<prad_buf_t> alone;  // views that do not start on a 16-byte boundary get a launch of their own
    for (int32_t i = 0; i < n; ++i) {
        REQUIRE_BUF(bufs[i]);
        if (reinterpret_cast<uintptr_t>(bufs[i]->ptr) % 16 != 0) { alone.push_back(bufs[i]); continue; }
        ptrs.push_back(bufs[i]->ptr);
        bytes.push_back((size_t)count(bufs[i]) * (bufs[i]->dtype == PRAD_F64 ? 8 : 4));
    }
    ENQUEUE_LOCK();
    HIP_TRY(prad::launch_fill_zero_multi(ptrs.data(), bytes.data(), (int)ptrs.size(), CUR_STREAM), PRAD_ERR_LAUNCH);
    for (prad_buf_t b : alone) {
        if (b->dtype == PRAD_F64) HIP_TRY(launch_fill_zero<double>(static_cast<double*>(b->ptr), count(b), CUR_STREAM), PRAD_ERR_LAUNCH);
        else HIP_TRY(launch_fill_zero<float>(static_cast<float*>(b->ptr), count(b), CUR_STREAM), PRAD_ERR_LAUNCH);
    }
    return PRAD_OK;
}

int32_t prad_buf_upload_rows(prad_buf_t b, const void* const* row_ptrs, const int64_t* row_lengths) {
    REQUIRE_INIT();
    REQUIRE_BUF(b);
    if (row_ptrs == nullptr) return fail(PRAD_ERR_ARG, "row_ptrs is NULL");
    const int64_t nrows = b->depth * b->rows;
    if (row_lengths)
        for (int64_t i = 0; i < nrows; ++i)
            if (row_lengths[i] != b->cols) return fail(PRAD_ERR_NOT_RECTANGULAR, "The given jagged array is not rectangular.");
    for (int64_t i = 0; i < nrows; ++i)
        if (row_ptrs[i] == nullptr) return fail(PRAD_ERR_NOT_RECTANGULAR, "The given jagged array is not rectangular.");
    const size_t row_bytes = (size_t)b->cols * elem_size(b->dtype);
    ENQUEUE_LOCK();
    NOT_WHILE_RECORDING("a copy to or from the host");
    int64_t rows_per_chunk = (int64_t)(STAGING_CHUNK / row_bytes);
    if (rows_per_chunk < 1) rows_per_chunk = 1;
    if (rows_per_chunk > nrows) rows_per_chunk = nrows;
    if (int32_t st = ensure_pinned((size_t)rows_per_chunk * row_bytes)) return st;
    for (int64_t r0 = 0; r0 < nrows; r0 += rows_per_chunk) {
        const int64_t nr = nrows - r0 < rows_per_chunk ? nrows - r0 : rows_per_chunk;
        char* stage = static_cast<char*>(g_ctx.pinned);
        for (int64_t i = 0; i < nr; ++i) memcpy(stage + (size_t)i * row_bytes, row_ptrs[r0 + i], row_bytes);
        HIP_TRY(hipMemcpyAsync(static_cast<char*>(b->ptr) + (size_t)r0 * row_bytes, stage, (size_t)nr * row_bytes,
                               hipMemcpyHostToDevice, g_ctx.stream), PRAD_ERR_LAUNCH);
        ++g_ctx.stat_stream_syncs;
        HIP_TRY(hipStreamSynchronize(g_ctx.stream), PRAD_ERR_LAUNCH);
    }
    return PRAD_OK;
}

int32_t prad_buf_download_rows(prad_buf_t b, void* const* row_ptrs) {
    REQUIRE_INIT();
    REQUIRE_BUF(b);
    if (row_ptrs == nullptr) return fail(PRAD_ERR_ARG, "row_ptrs is NULL");
    const int64_t nrows = b->depth * b->rows;
    for (int64_t i = 0; i < nrows; ++i)
        if (row_ptrs[i] == nullptr) return fail(PRAD_ERR_NOT_RECTANGULAR, "The given jagged array is not rectangular.");
    const size_t row_bytes = (size_t)b->cols * elem_size(b->dtype);
    ENQUEUE_LOCK();
    NOT_WHILE_RECORDING("a copy to or from the host");
    int64_t rows_per_chunk = (int64_t)(STAGING_CHUNK / row_bytes);
    if (rows_per_chunk < 1) rows_per_chunk = 1;
    if (rows_per_chunk > nrows) rows_per_chunk = nrows;
    if (int32_t st = ensure_pinned((size_t)rows_per_chunk * row_bytes)) return st;
    for (int64_t r0 = 0; r0 < nrows; r0 += rows_per_chunk) {
        const int64_t nr = nrows - r0 < rows_per_chunk ? nrows - r0 : rows_per_chunk;
        char* stage = static_cast<char*>(g_ctx.pinned);
        HIP_TRY(hipMemcpyAsync(stage, static_cast<char*>(b->ptr) + (size_t)r0 * row_bytes, (size_t)nr * row_bytes,
                               hipMemcpyDeviceToHost, g_ctx.stream), PRAD_ERR_LAUNCH);
        ++g_ctx.stat_stream_syncs;
        HIP_TRY(hipStreamSynchronize(g_ctx.stream), PRAD_ERR_LAUNCH);
        for (int64_t i = 0; i < nr; ++i) memcpy(row_ptrs[r0 + i], stage + (size_t)i * row_bytes, row_bytes);
    }
    return PRAD_OK;
}

int32_t prad_buf_upload(prad_buf_t b, const void* src, int64_t ld) {
    REQUIRE_INIT();
    REQUIRE_BUF(b);
    if (src == nullptr || ld < b->cols) return fail(PRAD_ERR_ARG, "bad source pointer or leading dimension");
    const size_t es = elem_size(b->dtype);
    ENQUEUE_LOCK();
    NOT_WHILE_RECORDING("a copy to or from the host");
    HIP_TRY(hipMemcpy2DAsync(b->ptr, (size_t)b->cols * es, src, (size_t)ld * es, (size_t)b->cols * es,
                             (size_t)(b->depth * b->rows), hipMemcpyHostToDevice, g_ctx.stream), PRAD_ERR_LAUNCH);
    ++g_ctx.stat_stream_syncs;
    HIP_TRY(hipStreamSynchronize(g_ctx.stream), PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

int32_t prad_buf_download(prad_buf_t b, void* dst, int64_t ld) {
    REQUIRE_INIT();
    REQUIRE_BUF(b);
    if (dst == nullptr || ld < b->cols) return fail(PRAD_ERR_ARG, "bad destination pointer or leading dimension");
    const size_t es = elem_size(b->dtype);
    ENQUEUE_LOCK();
    NOT_WHILE_RECORDING("a copy to or from the host");
    HIP_TRY(hipMemcpy2DAsync(dst, (size_t)ld * es, b->ptr, (size_t)b->cols * es, (size_t)b->cols * es,
                             (size_t)(b->depth * b->rows), hipMemcpyDeviceToHost, g_ctx.stream), PRAD_ERR_LAUNCH);
    ++g_ctx.stat_stream_syncs;
    HIP_TRY(hipStreamSynchronize(g_ctx.stream), PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

int32_t prad_buf_copy(prad_buf_t dst, prad_buf_t src) {
    REQUIRE_INIT();
    REQUIRE_BUF(dst); REQUIRE_BUF(src);
    if (int32_t st = same_dtype({dst, src})) return st;
    if (int32_t st = same_shape(dst, src, "copy")) return st;
    ENQUEUE_LOCK();
    // A kernel rather than hipMemcpyAsync: it can be recorded into a captured graph and shows up in
    // kernel traces as a plain copy of known size.
    if (src->dtype == PRAD_F64)
        HIP_TRY(launch_copy<double>(static_cast<double*>(dst->ptr), static_cast<const double*>(src->ptr), count(src), CUR_STREAM),
                PRAD_ERR_LAUNCH);
    else
        HIP_TRY(launch_copy<float>(static_cast<float*>(dst->ptr), static_cast<const float*>(src->ptr), count(src), CUR_STREAM),
                PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

// ---------------------------------------------------------------------------------------------
int32_t prad_gemm(int32_t transA, int32_t transB, prad_buf_t A, prad_buf_t B, prad_buf_t C, int32_t accumulate) {
    REQUIRE_INIT();
    ENQUEUE_LOCK();
    return enqueue_gemm(transA, transB, A, B, C, accumulate, Epilogue{}, false);
}

int32_t prad_gemm_batched(int32_t transA, int32_t transB, prad_buf_t A, prad_buf_t B, prad_buf_t C, int32_t accumulate) {
    REQUIRE_INIT();
    ENQUEUE_LOCK();
    return enqueue_gemm(transA, transB, A, B, C, accumulate, Epilogue{}, true);
}

int32_t prad_matmul_fwd(prad_buf_t A, prad_buf_t B, prad_buf_t C) {
    REQUIRE_INIT();
    ENQUEUE_LOCK();
    return enqueue_gemm(0, 0, A, B, C, 0, Epilogue{}, false);
}

int32_t prad_matmul_fwd_fused(prad_buf_t A, prad_buf_t B, prad_buf_t bias, prad_buf_t Z, prad_buf_t H, int32_t act, double alpha) {
    REQUIRE_INIT();
    if (bias != nullptr) REQUIRE_BUF(bias);
    if (Z != nullptr) REQUIRE_BUF(Z);
    Epilogue ep;
    ep.bias = bias; ep.Z = Z; ep.act_fwd = act; ep.alpha = alpha;
    ENQUEUE_LOCK();
    return enqueue_gemm(0, 0, A, B, H, 0, ep, false);
}

// Bias gradient by its own launch(es); lock held, handles validated by the caller.
static int32_t matmul_bwd_bias_only_locked(prad_buf_t dC, prad_buf_t dbias) {
    REQUIRE_BUF(dbias);
    if (dbias->dtype != dC->dtype) return fail(PRAD_ERR_DTYPE, "buffers of different element types in one call");
    if (dbias->cols != dC->cols || dbias->rows != 1 || dbias->depth != 1 || dC->depth != 1)
        return fail(PRAD_ERR_ARG, "bias gradient must be 1 x cols");
    double* ws = nullptr;
    if (colsum_chunks(dC->rows) > 1) {
        if (int32_t st = ensure_workspace((size_t)colsum_chunks(dC->rows) * dC->cols * sizeof(double))) return st;
        ws = static_cast<double*>(CUR_WORKSPACE);
    }
    if (dC->dtype == PRAD_F64)
        HIP_TRY(launch_colsum<double>(static_cast<const double*>(dC->ptr), static_cast<double*>(dbias->ptr), dC->rows, dC->cols, ws,
                                      CUR_STREAM), PRAD_ERR_LAUNCH);
    else
        HIP_TRY(launch_colsum<float>(static_cast<const float*>(dC->ptr), static_cast<float*>(dbias->ptr), dC->rows, dC->cols, ws,
                                     CUR_STREAM), PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

static int32_t matmul_bwd_locked(prad_buf_t dC, prad_buf_t A, prad_buf_t B, prad_buf_t dA, prad_buf_t dB, int32_t acc_dA,
                                 int32_t acc_dB, const Epilogue& ep, prad_buf_t dbias = nullptr) {
    REQUIRE_BUF(dC); REQUIRE_BUF(A); REQUIRE_BUF(B);
    if (dbias != nullptr) {
        REQUIRE_BUF(dbias);
        if (dbias->dtype != dC->dtype) return fail(PRAD_ERR_DTYPE, "buffers of different element types in one call");
        if (dbias->cols != dC->cols || dbias->rows != 1 || dbias->depth != 1 || dC->depth != 1)
            return fail(PRAD_ERR_ARG, "bias gradient must be 1 x cols");
    }
    if (A->cols != B->rows) return fail(PRAD_ERR_SHAPE, "Input 1 columns do not match Input 2 rows");
    if (dC->rows != A->rows || dC->cols != B->cols)
        return fail(PRAD_ERR_ARG, "upstream gradient is %lldx%lld, the product is %lldx%lld", (long long)dC->rows,
                    (long long)dC->cols, (long long)A->rows, (long long)B->cols);
    Epilogue rider;
    if (dB != nullptr && dbias != nullptr && dC->rows < COLSUM_CHUNK_ROWS) { rider.colsum_src = dC; rider.colsum_dst = dbias; }
    if (dB != nullptr && dbias != nullptr && rider.colsum_dst == nullptr && dC->dtype == PRAD_F32 && valid(dB) && valid(dbias)) {
        // a tall dC whose weight gradient runs as one pass over A and dC: the column sums are taken in that pass
        Epilogue tall;
        tall.colsum_src = dC; tall.colsum_dst = dbias;
        if (gemm_skinny_eligible(gemm_args_of<float>(1, 0, A, dC, dB, acc_dB, tall, false))) rider = tall;
    }
    bool paired = false;
    // (one launch only if the first product's output is not an operand of the second: launched one after the other,
    // the second would read what the first wrote)
    auto overlap = [](prad_buf_t x, prad_buf_t y) {
        const char* x0 = static_cast<const char*>(x->ptr);
        const char* y0 = static_cast<const char*>(y->ptr);
        const size_t xb = (size_t)count(x) * elem_size(x->dtype), yb = (size_t)count(y) * elem_size(y->dtype);
        return x0 < y0 + yb && y0 < x0 + xb;
    };
    if (dA != nullptr && dB != nullptr && valid(dA) && valid(dB) && !overlap(dA, dC) && !overlap(dA, A) && !overlap(dA, dB) &&
        !overlap(dB, dC) && !overlap(dB, B) && (dbias == nullptr || !overlap(dbias, dA))) {
        if (int32_t st = validate_gemm(0, 1, dC, B, dA, ep, false)) return st;
        if (int32_t st = validate_gemm(1, 0, A, dC, dB, rider, false)) return st;
        if (int32_t st = dC->dtype == PRAD_F64
                             ? enqueue_gradient_pair_t<double>(dC, A, B, dA, dB, acc_dA, acc_dB, ep, rider, &paired)
                             : enqueue_gradient_pair_t<float>(dC, A, B, dA, dB, acc_dA, acc_dB, ep, rider, &paired))
            return st;
    }
    if (dA != nullptr && !paired) {
        if (int32_t st = enqueue_gemm(0, 1, dC, B, dA, acc_dA, ep, false)) return st;  // dA = dC . B^T
    }
    if (dB != nullptr && !paired) {
        if (int32_t st = enqueue_gemm(1, 0, A, dC, dB, acc_dB, rider, false)) return st;  // dB = A^T . dC
    }
    if (rider.colsum_dst != nullptr) dbias = nullptr;
    if (dbias != nullptr) return matmul_bwd_bias_only_locked(dC, dbias);  // nothing to ride along with, or a tall matrix
    return PRAD_OK;
}

int32_t prad_matmul_bwd(prad_buf_t dC, prad_buf_t A, prad_buf_t B, prad_buf_t dA, prad_buf_t dB, int32_t accumulate_dA,
                        int32_t accumulate_dB) {
    REQUIRE_INIT();
    ENQUEUE_LOCK();
    return matmul_bwd_locked(dC, A, B, dA, dB, accumulate_dA, accumulate_dB, Epilogue{});
}

int32_t prad_matmul_bwd_fused(prad_buf_t dC, prad_buf_t A, prad_buf_t B, prad_buf_t dA, prad_buf_t dB, int32_t accumulate_dB,
                              int32_t act, prad_buf_t act_src, double alpha) {
    REQUIRE_INIT();
    Epilogue ep;
    ep.act_bwd = act; ep.act_src = act_src; ep.alpha = alpha;
    ENQUEUE_LOCK();
    return matmul_bwd_locked(dC, A, B, dA, dB, 0, accumulate_dB, ep);
}

int32_t prad_matmul_batch_sum_fwd(prad_buf_t A, prad_buf_t B, prad_buf_t bias, prad_buf_t C) {
    REQUIRE_INIT();
    REQUIRE_BUF(A); REQUIRE_BUF(B); REQUIRE_BUF(C);
    if (bias != nullptr) REQUIRE_BUF(bias);
    if (int32_t st = same_dtype({A, B, bias, C})) return st;
    if (A->depth != B->depth || A->depth > 65535) return fail(PRAD_ERR_SHAPE, "both operands must hold the same number of slices");
    if (A->cols != B->rows) return fail(PRAD_ERR_SHAPE, "Input 1 columns do not match Input 2 rows");
    if (C->depth != 1 || C->rows != A->rows || C->cols != B->cols)
        return fail(PRAD_ERR_ARG, "output must be %lldx%lld", (long long)A->rows, (long long)B->cols);
    if (bias && (bias->rows != 1 || bias->cols != C->cols || bias->depth != 1))
        return fail(PRAD_ERR_ARG, "The length of the bias vector must be the same as the number of columns in the input matrix.");
    ENQUEUE_LOCK();
    return A->dtype == PRAD_F64 ? batch_sum_fwd_t<double>(A, B, bias, C) : batch_sum_fwd_t<float>(A, B, bias, C);
}

int32_t prad_matmul_batch_sum_bwd(prad_buf_t dC, prad_buf_t A, prad_buf_t B, prad_buf_t dA, prad_buf_t dB, prad_buf_t dbias) {
    REQUIRE_INIT();
    REQUIRE_BUF(dC); REQUIRE_BUF(A); REQUIRE_BUF(B);
    if (A->depth != B->depth) return fail(PRAD_ERR_SHAPE, "both operands must hold the same number of slices");
    if (A->cols != B->rows) return fail(PRAD_ERR_SHAPE, "Input 1 columns do not match Input 2 rows");
    if (dC->depth != 1 || dC->rows != A->rows || dC->cols != B->cols)
        return fail(PRAD_ERR_ARG, "upstream gradient is %lldx%lld, the product is %lldx%lld", (long long)dC->rows,
                    (long long)dC->cols, (long long)A->rows, (long long)B->cols);
    ENQUEUE_LOCK();
    if (dA != nullptr) {
        REQUIRE_BUF(dA);
        if (int32_t st = same_shape(A, dA, "gradient of the first operand")) return st;
        if (int32_t st = enqueue_gemm(0, 1, dC, B, dA, 0, Epilogue{}, true)) return st;  // dA[q] = dC . B[q]^T
    }
    if (dB != nullptr) {
        REQUIRE_BUF(dB);
        if (int32_t st = same_shape(B, dB, "gradient of the second operand")) return st;
        if (int32_t st = enqueue_gemm(1, 0, A, dC, dB, 0, Epilogue{}, true)) return st;  // dB[q] = A[q]^T . dC
    }
    if (dbias != nullptr) return matmul_bwd_bias_only_locked(dC, dbias);
    return PRAD_OK;
}

int32_t prad_matmul_bias_bwd(prad_buf_t dC, prad_buf_t A, prad_buf_t B, prad_buf_t dA, prad_buf_t dB, prad_buf_t dbias,
                             int32_t accumulate_dB, int32_t act, prad_buf_t act_src, double alpha) {
    REQUIRE_INIT();
    Epilogue ep;
    ep.act_bwd = act; ep.act_src = act_src; ep.alpha = alpha;
    ENQUEUE_LOCK();
    return matmul_bwd_locked(dC, A, B, dA, dB, 0, accumulate_dB, ep, dbias);
}

#define RAW_GEMM(SFX, T)                                                                                              \
    int32_t prad_gemm_##SFX(int32_t transA, int32_t transB, int64_t M, int64_t N, int64_t K, const T* A, int64_t lda, \
                            const T* B, int64_t ldb, T* C, int64_t ldc, int32_t accumulate) {                         \
        REQUIRE_INIT();                                                                                               \
        if (A == nullptr || B == nullptr || C == nullptr) return fail(PRAD_ERR_ARG, "NULL matrix pointer");           \
        if (M < 0 || N < 0 || K < 0) return fail(PRAD_ERR_ARG, "negative dimension");                                 \
        if ((transA != 0 && transA != 1) || (transB != 0 && transB != 1) || (transA && transB))                       \
            return fail(PRAD_ERR_ARG, "unsupported transpose combination (%d, %d)", transA, transB);                  \
        if (lda < (transA ? M : K) || ldb < (transB ? K : N) || ldc < N) return fail(PRAD_ERR_ARG, "leading dimension too small"); \
        GemmArgs<T> a = plain_gemm<T>(transA, transB, M, N, K, A, lda, B, ldb, C, ldc, accumulate);                   \
        ENQUEUE_LOCK();                                                                                               \
        if (int32_t st = attach_split_workspace(a)) return st;                                                        \
        HIP_TRY(launch_gemm<T>(a, CUR_STREAM), PRAD_ERR_LAUNCH);                                                    \
        return PRAD_OK;                                                                                               \
    }
RAW_GEMM(f64, double)
RAW_GEMM(f32, float)

#define RAW_BATCHED_GEMM(SFX, T)                                                                                       \
    int32_t prad_gemm_strided_batched_##SFX(int32_t transA, int32_t transB, int64_t M, int64_t N, int64_t K, const T* A, \
                                            int64_t lda, int64_t strideA, const T* B, int64_t ldb, int64_t strideB, T* C, \
                                            int64_t ldc, int64_t strideC, int32_t batch, int32_t accumulate) {         \
        REQUIRE_INIT();                                                                                                \
        if (A == nullptr || B == nullptr || C == nullptr) return fail(PRAD_ERR_ARG, "NULL matrix pointer");            \
        if (M < 0 || N < 0 || K < 0 || batch < 0 || strideA < 0 || strideB < 0 || strideC < 0)                         \
            return fail(PRAD_ERR_ARG, "negative dimension");                                                           \
        if ((transA != 0 && transA != 1) || (transB != 0 && transB != 1) || (transA && transB))                        \
            return fail(PRAD_ERR_ARG, "unsupported transpose combination (%d, %d)", transA, transB);                   \
        if (lda < (transA ? M : K) || ldb < (transB ? K : N) || ldc < N) return fail(PRAD_ERR_ARG, "leading dimension too small"); \
        if (batch > 1 && strideC < (M - 1) * ldc + N) return fail(PRAD_ERR_ARG, "outputs of different products overlap"); \
        if (batch > 65535) return fail(PRAD_ERR_ARG, "at most 65535 products per call");                               \
        GemmArgs<T> a = plain_gemm<T>(transA, transB, M, N, K, A, lda, B, ldb, C, ldc, accumulate);                    \
        a.batch = batch; a.strideA = strideA; a.strideB = strideB; a.strideC = strideC;                                \
        ENQUEUE_LOCK();                                                                                                \
        HIP_TRY(launch_gemm<T>(a, CUR_STREAM), PRAD_ERR_LAUNCH);                                                     \
        return PRAD_OK;                                                                                                \
    }
RAW_BATCHED_GEMM(f64, double)
RAW_BATCHED_GEMM(f32, float)

#define RAW_BATCHED_GEMM_2D(SFX, T)                                                                                    \
    int32_t prad_gemm_strided_batched_2d_##SFX(int32_t transA, int32_t transB, int64_t M, int64_t N, int64_t K, const T* A, \
                                               int64_t lda, int64_t strideA, int64_t istrideA, const T* B, int64_t ldb,  \
                                               int64_t strideB, int64_t istrideB, T* C, int64_t ldc, int64_t strideC,    \
                                               int64_t istrideC, int32_t batch_outer, int32_t batch_inner, int32_t accumulate) { \
        REQUIRE_INIT();                                                                                                \
        if (A == nullptr || B == nullptr || C == nullptr) return fail(PRAD_ERR_ARG, "NULL matrix pointer");            \
        if (M < 0 || N < 0 || K < 0 || batch_outer < 0 || batch_inner < 1 || strideA < 0 || strideB < 0 || strideC < 0 || \
            istrideA < 0 || istrideB < 0 || istrideC < 0)                                                              \
            return fail(PRAD_ERR_ARG, "negative dimension");                                                           \
        if ((transA != 0 && transA != 1) || (transB != 0 && transB != 1) || (transA && transB))                        \
            return fail(PRAD_ERR_ARG, "unsupported transpose combination (%d, %d)", transA, transB);                   \
        if (lda < (transA ? M : K) || ldb < (transB ? K : N) || ldc < N) return fail(PRAD_ERR_ARG, "leading dimension too small"); \
        if ((int64_t)batch_outer * batch_inner > 65535) return fail(PRAD_ERR_ARG, "at most 65535 products per call");  \
        GemmArgs<T> a = plain_gemm<T>(transA, transB, M, N, K, A, lda, B, ldb, C, ldc, accumulate);                    \
        a.batch = batch_outer * batch_inner; a.strideA = strideA; a.strideB = strideB; a.strideC = strideC;            \
        a.batch_inner = batch_inner; a.istrideA = istrideA; a.istrideB = istrideB; a.istrideC = istrideC;              \
        ENQUEUE_LOCK();                                                                                                \
        HIP_TRY(launch_gemm<T>(a, CUR_STREAM), PRAD_ERR_LAUNCH);                                                     \
        return PRAD_OK;                                                                                                \
    }
RAW_BATCHED_GEMM_2D(f64, double)
RAW_BATCHED_GEMM_2D(f32, float)

// ---------------------------------------------------------------------------------------------
int32_t prad_matmul_fwd_host(int32_t dtype, const void* const* a_rows, const void* const* b_rows, void* const* c_rows, int64_t M,
                             int64_t K, int64_t K2, int64_t N) {
    REQUIRE_INIT();
    if (K != K2) return fail(PRAD_ERR_SHAPE, "Input 1 columns do not match Input 2 rows");
    prad_buf_t A = nullptr, B = nullptr, C = nullptr;
    int32_t st = prad_buf_alloc(dtype, M, K, &A);
    if (!st) st = prad_buf_alloc(dtype, K, N, &B);
    if (!st) st = prad_buf_alloc(dtype, M, N, &C);
    if (!st) st = prad_buf_upload_rows(A, a_rows, nullptr);
    if (!st) st = prad_buf_upload_rows(B, b_rows, nullptr);
    if (!st) st = prad_matmul_fwd(A, B, C);
    if (!st) st = prad_buf_download_rows(C, c_rows);
    std::string keep = tl_error;
    prad_buf_free(A); prad_buf_free(B); prad_buf_free(C);
    if (st) tl_error = keep;
    return st;
}

int32_t prad_matmul_bwd_host(int32_t dtype, const void* const* dc_rows, const void* const* a_rows, const void* const* b_rows,
                             void* const* da_rows, void* const* db_rows, int64_t M, int64_t K, int64_t N) {
    REQUIRE_INIT();
    prad_buf_t dC = nullptr, A = nullptr, B = nullptr, dA = nullptr, dB = nullptr;
    int32_t st = prad_buf_alloc(dtype, M, N, &dC);
    if (!st) st = prad_buf_alloc(dtype, M, K, &A);
    if (!st) st = prad_buf_alloc(dtype, K, N, &B);
    if (!st) st = prad_buf_alloc(dtype, M, K, &dA);
    if (!st) st = prad_buf_alloc(dtype, K, N, &dB);
    if (!st) st = prad_buf_upload_rows(dC, dc_rows, nullptr);
    if (!st) st = prad_buf_upload_rows(A, a_rows, nullptr);
    if (!st) st = prad_buf_upload_rows(B, b_rows, nullptr);
    if (!st) st = prad_matmul_bwd(dC, A, B, dA, dB, 0, 0);
    if (!st) st = prad_buf_download_rows(dA, da_rows);
    if (!st) st = prad_buf_download_rows(dB, db_rows);
    std::string keep = tl_error;
    prad_buf_free(dC); prad_buf_free(A); prad_buf_free(B); prad_buf_free(dA); prad_buf_free(dB);
    if (st) tl_error = keep;
    return st;
}

// The tape engine's products on flat row-major host arrays: Tensor.MatrixMultiply (src/PRAD/Tensor.cs:572-608,
// which hands the arrays to a BLAS gemm) and TensorReverse.MatrixMultiplyReverse (src/PRAD/TensorReverse.cs:94-157).
int32_t prad_tensor_matmul_host(int32_t dtype, const void* a, const void* b, void* c, int64_t m, int64_t k, int64_t k2, int64_t n,
                                double alpha) {
    REQUIRE_INIT();
    if (k != k2) return fail(PRAD_ERR_SHAPE, "Incompatible shapes for matrix multiplication.");
    if (m < 0 || k < 0 || n < 0 || a == nullptr || b == nullptr || c == nullptr) return fail(PRAD_ERR_ARG, "bad tensor arguments");
    prad_buf_t A = nullptr, B = nullptr, C = nullptr;
    int32_t st = prad_buf_alloc(dtype, m, k, &A);
    if (!st) st = prad_buf_alloc(dtype, k, n, &B);
    if (!st) st = prad_buf_alloc(dtype, m, n, &C);
    if (!st) st = prad_buf_upload(A, a, k);
    if (!st) st = prad_buf_upload(B, b, n);
    if (!st) st = prad_matmul_fwd(A, B, C);
    if (!st && alpha != 1.0) st = prad_scale(C, C, alpha);
    if (!st) st = prad_buf_download(C, c, n);
    std::string keep = tl_error;
    prad_buf_free(A); prad_buf_free(B); prad_buf_free(C);
    if (st) tl_error = keep;
    return st;
}

int32_t prad_tensor_matmul_reverse_host(int32_t dtype, const void* dc, const void* a, const void* b, void* da, void* db, int64_t m,
                                        int64_t k, int64_t n) {
    REQUIRE_INIT();
    if (m < 0 || k < 0 || n < 0 || dc == nullptr || a == nullptr || b == nullptr || da == nullptr || db == nullptr)
        return fail(PRAD_ERR_ARG, "bad tensor arguments");
    prad_buf_t dC = nullptr, A = nullptr, B = nullptr, dA = nullptr, dB = nullptr;
    int32_t st = prad_buf_alloc(dtype, m, n, &dC);
    if (!st) st = prad_buf_alloc(dtype, m, k, &A);
    if (!st) st = prad_buf_alloc(dtype, k, n, &B);
    if (!st) st = prad_buf_alloc(dtype, m, k, &dA);
    if (!st) st = prad_buf_alloc(dtype, k, n, &dB);
    if (!st) st = prad_buf_upload(dC, dc, n);
    if (!st) st = prad_buf_upload(A, a, k);
    if (!st) st = prad_buf_upload(B, b, n);
    if (!st) st = prad_matmul_bwd(dC, A, B, dA, dB, 0, 0);
    if (!st) st = prad_buf_download(dA, da, k);
    if (!st) st = prad_buf_download(dB, db, n);
    std::string keep = tl_error;
    prad_buf_free(dC); prad_buf_free(A); prad_buf_free(B); prad_buf_free(dA); prad_buf_free(dB);
    if (st) tl_error = keep;
    return st;
}

// ---------------------------------------------------------------------------------------------
int32_t prad_matmul_sum_fwd(prad_buf_t A, prad_buf_t B, prad_buf_t out) {
    REQUIRE_INIT();
    REQUIRE_BUF(A); REQUIRE_BUF(B); REQUIRE_BUF(out);
    if (int32_t st = same_dtype({A, B, out})) return st;
    if (A->cols != B->rows) return fail(PRAD_ERR_SHAPE, "Matrix dimensions must be compatible for multiplication.");
    const int64_t P = B->depth, S = A->depth;
    if (out->depth != S || out->rows != 1 || out->cols != P)
        return fail(PRAD_ERR_ARG, "output must be 1 x depth(B) for each of the depth(A) samples");
    if (S * P > 65535) return fail(PRAD_ERR_ARG, "at most 65535 products per call");
    ENQUEUE_LOCK();
    const size_t ws = (size_t)S * P * gemm_tiles_per_product(A->rows, B->cols) * sizeof(double);
    if (int32_t st = ensure_workspace(ws)) return st;
    double* w = static_cast<double*>(CUR_WORKSPACE);
    if (A->dtype == PRAD_F64)
        HIP_TRY(launch_matmul_sum_fwd<double>(static_cast<const double*>(A->ptr), static_cast<const double*>(B->ptr),
                                              static_cast<double*>(out->ptr), w, A->rows, A->cols, B->cols, P, S, CUR_STREAM),
                PRAD_ERR_LAUNCH);
    else
        HIP_TRY(launch_matmul_sum_fwd<float>(static_cast<const float*>(A->ptr), static_cast<const float*>(B->ptr),
                                             static_cast<float*>(out->ptr), w, A->rows, A->cols, B->cols, P, S, CUR_STREAM),
                PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

int32_t prad_matmul_sum_bwd(prad_buf_t A, prad_buf_t B, prad_buf_t dOut, prad_buf_t dA, prad_buf_t dB) {
    REQUIRE_INIT();
    REQUIRE_BUF(A); REQUIRE_BUF(B); REQUIRE_BUF(dOut);
    if (dA != nullptr) REQUIRE_BUF(dA);
    if (dB != nullptr) REQUIRE_BUF(dB);
    if (int32_t st = same_dtype({A, B, dOut, dA, dB})) return st;
    const int64_t M = A->rows, K = A->cols, N = B->cols, P = B->depth, S = A->depth;
    if (B->rows != K) return fail(PRAD_ERR_SHAPE, "Matrix dimensions must be compatible for multiplication.");
    if (dOut->depth != S || dOut->rows != 1 || dOut->cols != P)
        return fail(PRAD_ERR_ARG, "upstream gradient must be 1 x depth(B) for each of the depth(A) samples");
    if (S > 65535) return fail(PRAD_ERR_ARG, "at most 65535 samples per call");
    if (dA != nullptr) {
        if (N != M) return fail(PRAD_ERR_SHAPE, "transpose(B[q]) must have the shape of A (the reference adds them elementwise)");
        if (dA->depth != S || dA->rows != M || dA->cols != K) return fail(PRAD_ERR_ARG, "dA must have the shape of A");
    }
    if (dB != nullptr && (dB->depth != S * P || dB->rows != K || dB->cols != M))
        return fail(PRAD_ERR_ARG, "dB must be (samples * depth) x cols(A) x rows(A)");
    ENQUEUE_LOCK();
    if (A->dtype == PRAD_F64)
        HIP_TRY(launch_matmul_sum_bwd<double>(static_cast<const double*>(A->ptr), static_cast<const double*>(B->ptr),
                                              static_cast<const double*>(dOut->ptr), dA ? static_cast<double*>(dA->ptr) : nullptr,
                                              dB ? static_cast<double*>(dB->ptr) : nullptr, M, K, N, P, S, CUR_STREAM),
                PRAD_ERR_LAUNCH);
    else
        HIP_TRY(launch_matmul_sum_bwd<float>(static_cast<const float*>(A->ptr), static_cast<const float*>(B->ptr),
                                             static_cast<const float*>(dOut->ptr), dA ? static_cast<float*>(dA->ptr) : nullptr,
                                             dB ? static_cast<float*>(dB->ptr) : nullptr, M, K, N, P, S, CUR_STREAM),
                PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

// ---------------------------------------------------------------------------------------------
#define DISPATCH(b, call64, call32)                                  \
    do {                                                             \
        if ((b)->dtype == PRAD_F64) HIP_TRY(call64, PRAD_ERR_LAUNCH); \
        else HIP_TRY(call32, PRAD_ERR_LAUNCH);                       \
    } while (0)
#define D(b) static_cast<double*>((b)->ptr)
#define F(b) static_cast<float*>((b)->ptr)

int32_t prad_act_fwd(int32_t act, prad_buf_t x, prad_buf_t y, double alpha) {
    REQUIRE_INIT();
    REQUIRE_BUF(x); REQUIRE_BUF(y);
    if (act < PRAD_ACT_LEAKYRELU || act > PRAD_ACT_AMPLIFIED_SIGMOID) return fail(PRAD_ERR_ARG, "unknown activation selector");
    if (int32_t st = same_dtype({x, y})) return st;
    if (int32_t st = same_shape(x, y, "activation")) return st;
    ENQUEUE_LOCK();
    DISPATCH(x, launch_act_fwd<double>(act, D(x), D(y), count(x), alpha, CUR_STREAM),
             launch_act_fwd<float>(act, F(x), F(y), count(x), (float)alpha, CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_act_bwd(int32_t act, prad_buf_t src, prad_buf_t dy, prad_buf_t dx, double alpha) {
    REQUIRE_INIT();
    REQUIRE_BUF(src); REQUIRE_BUF(dy); REQUIRE_BUF(dx);
    if (act < PRAD_ACT_LEAKYRELU || act > PRAD_ACT_AMPLIFIED_SIGMOID) return fail(PRAD_ERR_ARG, "unknown activation selector");
    if (int32_t st = same_dtype({src, dy, dx})) return st;
    if (int32_t st = same_shape(src, dy, "activation backward")) return st;
    if (int32_t st = same_shape(src, dx, "activation backward")) return st;
    ENQUEUE_LOCK();
    DISPATCH(src, launch_act_bwd<double>(act, D(src), D(dy), D(dx), count(src), alpha, CUR_STREAM),
             launch_act_bwd<float>(act, F(src), F(dy), F(dx), count(src), (float)alpha, CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_hadamard_fwd(prad_buf_t a, prad_buf_t b, prad_buf_t y) {
    REQUIRE_INIT();
    REQUIRE_BUF(a); REQUIRE_BUF(b); REQUIRE_BUF(y);
    if (int32_t st = same_dtype({a, b, y})) return st;
    if (int32_t st = same_shape(a, b, "Hadamard product")) return st;
    if (int32_t st = same_shape(a, y, "Hadamard product")) return st;
    ENQUEUE_LOCK();
    DISPATCH(a, launch_hadamard_fwd<double>(D(a), D(b), D(y), count(a), CUR_STREAM),
             launch_hadamard_fwd<float>(F(a), F(b), F(y), count(a), CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_hadamard_bwd(prad_buf_t a, prad_buf_t b, prad_buf_t dy, prad_buf_t da, prad_buf_t db) {
    REQUIRE_INIT();
    REQUIRE_BUF(a); REQUIRE_BUF(b); REQUIRE_BUF(dy); REQUIRE_BUF(da); REQUIRE_BUF(db);
    if (int32_t st = same_dtype({a, b, dy, da, db})) return st;
    for (prad_buf_t o : {b, dy, da, db})
        if (int32_t st = same_shape(a, o, "Hadamard product")) return st;
    ENQUEUE_LOCK();
    DISPATCH(a, launch_hadamard_bwd<double>(D(a), D(b), D(dy), D(da), D(db), count(a), CUR_STREAM),
             launch_hadamard_bwd<float>(F(a), F(b), F(dy), F(da), F(db), count(a), CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_scale(prad_buf_t x, prad_buf_t y, double scalar) {
    REQUIRE_INIT();
    REQUIRE_BUF(x); REQUIRE_BUF(y);
    if (int32_t st = same_dtype({x, y})) return st;
    if (int32_t st = same_shape(x, y, "multiply by scalar")) return st;
    ENQUEUE_LOCK();
    DISPATCH(x, launch_scale<double>(D(y), D(x), count(x), scalar, CUR_STREAM),
             launch_scale<float>(F(y), F(x), count(x), (float)scalar, CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_accumulate(prad_buf_t dest, prad_buf_t grad) {
    REQUIRE_INIT();
    REQUIRE_BUF(dest); REQUIRE_BUF(grad);
    if (int32_t st = same_dtype({dest, grad})) return st;
    if (int32_t st = same_shape(dest, grad, "accumulate")) return st;
    ENQUEUE_LOCK();
    DISPATCH(dest, launch_accumulate<double>(D(dest), D(grad), count(dest), CUR_STREAM),
             launch_accumulate<float>(F(dest), F(grad), count(dest), CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_add(prad_buf_t a, prad_buf_t b, prad_buf_t y) {
    REQUIRE_INIT();
    REQUIRE_BUF(a); REQUIRE_BUF(b); REQUIRE_BUF(y);
    if (int32_t st = same_dtype({a, b, y})) return st;
    if (int32_t st = same_shape(a, b, "add")) return st;
    if (int32_t st = same_shape(a, y, "add")) return st;
    ENQUEUE_LOCK();
    DISPATCH(a, launch_add<double>(D(a), D(b), D(y), count(a), CUR_STREAM), launch_add<float>(F(a), F(b), F(y), count(a), CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_add_three(prad_buf_t a, prad_buf_t b, prad_buf_t c, prad_buf_t y) {
    REQUIRE_INIT();
    REQUIRE_BUF(a); REQUIRE_BUF(b); REQUIRE_BUF(c); REQUIRE_BUF(y);
    if (int32_t st = same_dtype({a, b, c, y})) return st;
    for (prad_buf_t o : {b, c, y})
        if (int32_t st = same_shape(a, o, "add three")) return st;
    ENQUEUE_LOCK();
    DISPATCH(a, launch_add_three<double>(D(a), D(b), D(c), D(y), count(a), CUR_STREAM),
             launch_add_three<float>(F(a), F(b), F(c), F(y), count(a), CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_transpose(prad_buf_t x, prad_buf_t y) {
    REQUIRE_INIT();
    REQUIRE_BUF(x); REQUIRE_BUF(y);
    if (int32_t st = same_dtype({x, y})) return st;
    if (x->depth != 1 || y->depth != 1 || y->rows != x->cols || y->cols != x->rows)
        return fail(PRAD_ERR_ARG, "the transpose of a %lldx%lld matrix is %lldx%lld", (long long)x->rows, (long long)x->cols,
                    (long long)x->cols, (long long)x->rows);
    if (x->ptr == y->ptr) return fail(PRAD_ERR_ARG, "transpose in place is not supported");
    ENQUEUE_LOCK();
    DISPATCH(x, launch_transpose<double>(D(x), D(y), x->rows, x->cols, CUR_STREAM),
             launch_transpose<float>(F(x), F(y), x->rows, x->cols, CUR_STREAM));
    return PRAD_OK;
}

static int32_t layernorm_shapes(prad_buf_t x, prad_buf_t mean, prad_buf_t stddev) {
    if (x->depth != 1) return fail(PRAD_ERR_SHAPE, "deep buffer passed to layer normalization");
    for (prad_buf_t o : {mean, stddev})
        if (o->depth != 1 || o->rows != 1 || o->cols != x->rows) return fail(PRAD_ERR_ARG, "mean and stddev must be 1 x rows");
    return PRAD_OK;
}

int32_t prad_layernorm_fwd(prad_buf_t x, prad_buf_t y, prad_buf_t mean, prad_buf_t stddev) {
    REQUIRE_INIT();
    REQUIRE_BUF(x); REQUIRE_BUF(y); REQUIRE_BUF(mean); REQUIRE_BUF(stddev);
    if (int32_t st = same_dtype({x, y, mean, stddev})) return st;
    if (int32_t st = same_shape(x, y, "layer normalization")) return st;
    if (int32_t st = layernorm_shapes(x, mean, stddev)) return st;
    ENQUEUE_LOCK();
    DISPATCH(x, launch_layernorm_fwd<double>(D(x), D(y), D(mean), D(stddev), x->rows, x->cols, CUR_STREAM),
             launch_layernorm_fwd<float>(F(x), F(y), F(mean), F(stddev), x->rows, x->cols, CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_layernorm_bwd(prad_buf_t x, prad_buf_t mean, prad_buf_t stddev, prad_buf_t dy, prad_buf_t dx) {
    REQUIRE_INIT();
    REQUIRE_BUF(x); REQUIRE_BUF(mean); REQUIRE_BUF(stddev); REQUIRE_BUF(dy); REQUIRE_BUF(dx);
    if (int32_t st = same_dtype({x, mean, stddev, dy, dx})) return st;
    if (int32_t st = same_shape(x, dy, "layer normalization backward")) return st;
    if (int32_t st = same_shape(x, dx, "layer normalization backward")) return st;
    if (int32_t st = layernorm_shapes(x, mean, stddev)) return st;
    ENQUEUE_LOCK();
    DISPATCH(x, launch_layernorm_bwd<double>(D(x), D(mean), D(stddev), D(dy), D(dx), x->rows, x->cols, CUR_STREAM),
             launch_layernorm_bwd<float>(F(x), F(mean), F(stddev), F(dy), F(dx), x->rows, x->cols, CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_add_broadcast_fwd(prad_buf_t x, prad_buf_t bias, prad_buf_t y) {
    REQUIRE_INIT();
    REQUIRE_BUF(x); REQUIRE_BUF(bias); REQUIRE_BUF(y);
    if (int32_t st = same_dtype({x, bias, y})) return st;
    if (bias->cols != x->cols || bias->rows != 1 || bias->depth != 1)
        return fail(PRAD_ERR_ARG, "The length of the bias vector must be the same as the number of columns in the input matrix.");
    if (int32_t st = same_shape(x, y, "add broadcasting")) return st;
    ENQUEUE_LOCK();
    DISPATCH(x, launch_add_broadcast_fwd<double>(D(x), D(bias), D(y), x->depth * x->rows, x->cols, CUR_STREAM),
             launch_add_broadcast_fwd<float>(F(x), F(bias), F(y), x->depth * x->rows, x->cols, CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_add_broadcast_bwd_bias(prad_buf_t dy, prad_buf_t dbias) {
    REQUIRE_INIT();
    REQUIRE_BUF(dy); REQUIRE_BUF(dbias);
    if (int32_t st = same_dtype({dy, dbias})) return st;
    if (dbias->cols != dy->cols || dbias->rows != 1 || dbias->depth != 1 || dy->depth != 1)
        return fail(PRAD_ERR_ARG, "bias gradient must be 1 x cols");
    ENQUEUE_LOCK();
    double* ws = nullptr;
    if (colsum_chunks(dy->rows) > 1) {
        if (int32_t st = ensure_workspace((size_t)colsum_chunks(dy->rows) * dy->cols * sizeof(double))) return st;
        ws = static_cast<double*>(CUR_WORKSPACE);
    }
    DISPATCH(dy, launch_colsum<double>(D(dy), D(dbias), dy->rows, dy->cols, ws, CUR_STREAM),
             launch_colsum<float>(F(dy), F(dbias), dy->rows, dy->cols, ws, CUR_STREAM));
    return PRAD_OK;
}

// ---------------------------------------------------------------------------------------------
static int32_t softmax_fwd_scaled(prad_buf_t x, double alpha, prad_buf_t y) {
    REQUIRE_INIT();
    REQUIRE_BUF(x); REQUIRE_BUF(y);
    if (int32_t st = same_dtype({x, y})) return st;
    if (int32_t st = same_shape(x, y, "softmax")) return st;
    ENQUEUE_LOCK();
    DISPATCH(x, launch_softmax_fwd<double>(D(x), D(y), x->depth * x->rows, x->cols, alpha, CUR_STREAM),
             launch_softmax_fwd<float>(F(x), F(y), x->depth * x->rows, x->cols, (float)alpha, CUR_STREAM));
    return PRAD_OK;
}

static int32_t softmax_bwd_scaled(prad_buf_t y, prad_buf_t dy, double alpha, prad_buf_t dx) {
    REQUIRE_INIT();
    REQUIRE_BUF(y); REQUIRE_BUF(dy); REQUIRE_BUF(dx);
    if (int32_t st = same_dtype({y, dy, dx})) return st;
    if (int32_t st = same_shape(y, dy, "softmax backward")) return st;
    if (int32_t st = same_shape(y, dx, "softmax backward")) return st;
    ENQUEUE_LOCK();
    DISPATCH(y, launch_softmax_bwd<double>(D(y), D(dy), D(dx), y->depth * y->rows, y->cols, alpha, CUR_STREAM),
             launch_softmax_bwd<float>(F(y), F(dy), F(dx), y->depth * y->rows, y->cols, (float)alpha, CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_softmax_fwd(prad_buf_t x, prad_buf_t y) { return softmax_fwd_scaled(x, 1.0, y); }
int32_t prad_softmax_bwd(prad_buf_t y, prad_buf_t dy, prad_buf_t dx) { return softmax_bwd_scaled(y, dy, 1.0, dx); }
int32_t prad_softmax_scaled_fwd(prad_buf_t x, double alpha, prad_buf_t y) { return softmax_fwd_scaled(x, alpha, y); }
int32_t prad_softmax_scaled_bwd(prad_buf_t y, prad_buf_t dy, double alpha, prad_buf_t dx) { return softmax_bwd_scaled(y, dy, alpha, dx); }

int32_t prad_cce_fwd(prad_buf_t p, prad_buf_t target, prad_buf_t loss) {
    REQUIRE_INIT();
    REQUIRE_BUF(p); REQUIRE_BUF(target); REQUIRE_BUF(loss);
    if (int32_t st = same_dtype({p, target, loss})) return st;
    if (p->depth != 1 || p->rows != target->rows || p->cols != target->cols || target->depth != 1)
        return fail(PRAD_ERR_ARG, "Output and target matrices must have the same dimensions.");
    if (loss->depth != 1 || loss->rows != 1 || loss->cols != 1) return fail(PRAD_ERR_ARG, "loss must be 1 x 1");
    ENQUEUE_LOCK();
    DISPATCH(p, launch_cce_fwd<double>(D(p), D(target), D(loss), p->rows, p->cols, CUR_STREAM),
             launch_cce_fwd<float>(F(p), F(target), F(loss), p->rows, p->cols, CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_cce_bwd(prad_buf_t p, prad_buf_t target, prad_buf_t dp) {
    REQUIRE_INIT();
    REQUIRE_BUF(p); REQUIRE_BUF(target); REQUIRE_BUF(dp);
    if (int32_t st = same_dtype({p, target, dp})) return st;
    if (p->depth != 1 || p->rows != target->rows || p->cols != target->cols || target->depth != 1)
        return fail(PRAD_ERR_ARG, "Output and target matrices must have the same dimensions.");
    if (int32_t st = same_shape(p, dp, "cross-entropy backward")) return st;
    ENQUEUE_LOCK();
    DISPATCH(p, launch_cce_bwd<double>(D(p), D(target), D(dp), p->rows, p->cols, CUR_STREAM),
             launch_cce_bwd<float>(F(p), F(target), F(dp), p->rows, p->cols, CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_mse_fwd(prad_buf_t y, prad_buf_t target, prad_buf_t loss) {
    REQUIRE_INIT();
    REQUIRE_BUF(y); REQUIRE_BUF(target); REQUIRE_BUF(loss);
    if (int32_t st = same_dtype({y, target, loss})) return st;
    if (y->depth != target->depth || y->rows != target->rows || y->cols != target->cols)
        return fail(PRAD_ERR_ARG, "Output and target matrices must have the same dimensions.");
    if (loss->depth != 1 || loss->rows != 1 || loss->cols != 1) return fail(PRAD_ERR_ARG, "loss must be 1 x 1");
    ENQUEUE_LOCK();
    if (int32_t st = ensure_workspace(mse_workspace_bytes())) return st;
    double* w = static_cast<double*>(CUR_WORKSPACE);
    DISPATCH(y, launch_mse_fwd<double>(D(y), D(target), D(loss), w, count(y), CUR_STREAM),
             launch_mse_fwd<float>(F(y), F(target), F(loss), w, count(y), CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_mse(prad_buf_t y, prad_buf_t target, prad_buf_t loss, prad_buf_t dy) {
    REQUIRE_INIT();
    REQUIRE_BUF(y); REQUIRE_BUF(target); REQUIRE_BUF(loss); REQUIRE_BUF(dy);
    if (int32_t st = same_dtype({y, target, loss, dy})) return st;
    if (y->depth != target->depth || y->rows != target->rows || y->cols != target->cols)
        return fail(PRAD_ERR_ARG, "Output and target matrices must have the same dimensions.");
    if (loss->depth != 1 || loss->rows != 1 || loss->cols != 1) return fail(PRAD_ERR_ARG, "loss must be 1 x 1");
    if (int32_t st = same_shape(y, dy, "mean squared error backward")) return st;
    ENQUEUE_LOCK();
    if (int32_t st = ensure_workspace(mse_workspace_bytes())) return st;
    double* w = static_cast<double*>(CUR_WORKSPACE);
    DISPATCH(y, launch_mse_fwd<double>(D(y), D(target), D(loss), w, count(y), CUR_STREAM, D(dy)),
             launch_mse_fwd<float>(F(y), F(target), F(loss), w, count(y), CUR_STREAM, F(dy)));
    return PRAD_OK;
}

int32_t prad_mse_bwd(prad_buf_t y, prad_buf_t target, prad_buf_t dy) {
    REQUIRE_INIT();
    REQUIRE_BUF(y); REQUIRE_BUF(target); REQUIRE_BUF(dy);
    if (int32_t st = same_dtype({y, target, dy})) return st;
    if (y->depth != target->depth || y->rows != target->rows || y->cols != target->cols)
        return fail(PRAD_ERR_ARG, "Output and target matrices must have the same dimensions.");
    if (int32_t st = same_shape(y, dy, "mean squared error backward")) return st;
    ENQUEUE_LOCK();
    DISPATCH(y, launch_mse_bwd<double>(D(y), D(target), D(dy), count(y), CUR_STREAM),
             launch_mse_bwd<float>(F(y), F(target), F(dy), count(y), CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_lstm_cell_fwd(prad_buf_t G, prad_buf_t c_prev, prad_buf_t c, prad_buf_t tanh_c, prad_buf_t h) {
    REQUIRE_INIT();
    REQUIRE_BUF(G); REQUIRE_BUF(c_prev); REQUIRE_BUF(c); REQUIRE_BUF(tanh_c); REQUIRE_BUF(h);
    if (int32_t st = same_dtype({G, c_prev, c, tanh_c, h})) return st;
    const int64_t rows = c->rows, hidden = c->cols;
    if (G->depth != 1 || c->depth != 1 || G->rows != rows || G->cols != 4 * hidden)
        return fail(PRAD_ERR_ARG, "gate pre-activations must be rows x 4*hidden");
    for (prad_buf_t o : {c_prev, tanh_c, h})
        if (int32_t st = same_shape(c, o, "LSTM cell")) return st;
    ENQUEUE_LOCK();
    DISPATCH(c, launch_lstm_cell_fwd<double>(D(G), D(c_prev), D(c), D(tanh_c), D(h), rows, hidden, CUR_STREAM),
             launch_lstm_cell_fwd<float>(F(G), F(c_prev), F(c), F(tanh_c), F(h), rows, hidden, CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_lstm_cell_bwd(prad_buf_t gates, prad_buf_t c_prev, prad_buf_t tanh_c, prad_buf_t dh_a, prad_buf_t dh_b, prad_buf_t dc_in,
                           prad_buf_t dG, prad_buf_t dc_prev) {
    REQUIRE_INIT();
    REQUIRE_BUF(gates); REQUIRE_BUF(c_prev); REQUIRE_BUF(tanh_c); REQUIRE_BUF(dh_a); REQUIRE_BUF(dG); REQUIRE_BUF(dc_prev);
    if (dh_b != nullptr) REQUIRE_BUF(dh_b);
    if (dc_in != nullptr) REQUIRE_BUF(dc_in);
    if (int32_t st = same_dtype({gates, c_prev, tanh_c, dh_a, dh_b, dc_in, dG, dc_prev})) return st;
    const int64_t rows = c_prev->rows, hidden = c_prev->cols;
    if (gates->rows != rows || gates->cols != 4 * hidden || c_prev->depth != 1 || gates->depth != 1)
        return fail(PRAD_ERR_ARG, "gates must be rows x 4*hidden");
    if (int32_t st = same_shape(gates, dG, "LSTM cell backward")) return st;
    for (prad_buf_t o : {tanh_c, dh_a, dh_b, dc_in, dc_prev})
        if (o != nullptr)
            if (int32_t st = same_shape(c_prev, o, "LSTM cell backward")) return st;
    ENQUEUE_LOCK();
    DISPATCH(c_prev,
             launch_lstm_cell_bwd<double>(D(gates), D(c_prev), D(tanh_c), D(dh_a), dh_b ? D(dh_b) : nullptr, dc_in ? D(dc_in) : nullptr,
                                          D(dG), D(dc_prev), rows, hidden, CUR_STREAM),
             launch_lstm_cell_bwd<float>(F(gates), F(c_prev), F(tanh_c), F(dh_a), dh_b ? F(dh_b) : nullptr, dc_in ? F(dc_in) : nullptr,
                                         F(dG), F(dc_prev), rows, hidden, CUR_STREAM));
    return PRAD_OK;
}

int32_t prad_lstm_step_fwd(prad_buf_t h_prev, prad_buf_t Wh, prad_buf_t G, prad_buf_t c_prev, prad_buf_t c, prad_buf_t tanh_c,
                           prad_buf_t h) {
    REQUIRE_INIT();
    REQUIRE_BUF(h_prev); REQUIRE_BUF(Wh); REQUIRE_BUF(G); REQUIRE_BUF(c_prev); REQUIRE_BUF(c); REQUIRE_BUF(tanh_c); REQUIRE_BUF(h);
    if (int32_t st = same_dtype({h_prev, Wh, G, c_prev, c, tanh_c, h})) return st;
    const int64_t rows = c->rows, hidden = c->cols;
    if (G->depth != 1 || c->depth != 1 || G->rows != rows || G->cols != 4 * hidden)
        return fail(PRAD_ERR_ARG, "gate pre-activations must be rows x 4*hidden");
    if (Wh->depth != 1 || Wh->rows != hidden || Wh->cols != 4 * hidden) return fail(PRAD_ERR_SHAPE, "recurrent weight must be hidden x 4*hidden");
    for (prad_buf_t o : {h_prev, c_prev, tanh_c, h})
        if (int32_t st = same_shape(c, o, "LSTM step")) return st;
    ENQUEUE_LOCK();
    return G->dtype == PRAD_F64 ? lstm_step_fwd_t<double>(h_prev, Wh, G, c_prev, c, tanh_c, h)
                                : lstm_step_fwd_t<float>(h_prev, Wh, G, c_prev, c, tanh_c, h);
}

int32_t prad_lstm_step_bwd(prad_buf_t dG_next, prad_buf_t Wh, prad_buf_t gates, prad_buf_t c_prev, prad_buf_t tanh_c,
                           prad_buf_t dh_loss, prad_buf_t dc_in, prad_buf_t dG, prad_buf_t dc_prev, prad_buf_t dh_scratch) {
    REQUIRE_INIT();
    REQUIRE_BUF(dG_next); REQUIRE_BUF(Wh); REQUIRE_BUF(gates); REQUIRE_BUF(c_prev); REQUIRE_BUF(tanh_c); REQUIRE_BUF(dh_loss);
    REQUIRE_BUF(dG); REQUIRE_BUF(dc_prev); REQUIRE_BUF(dh_scratch);
    if (dc_in != nullptr) REQUIRE_BUF(dc_in);
    if (int32_t st = same_dtype({dG_next, Wh, gates, c_prev, tanh_c, dh_loss, dc_in, dG, dc_prev, dh_scratch})) return st;
    const int64_t rows = c_prev->rows, hidden = c_prev->cols;
    if (gates->rows != rows || gates->cols != 4 * hidden || c_prev->depth != 1 || gates->depth != 1)
        return fail(PRAD_ERR_ARG, "gates must be rows x 4*hidden");
    if (Wh->depth != 1 || Wh->rows != hidden || Wh->cols != 4 * hidden) return fail(PRAD_ERR_SHAPE, "recurrent weight must be hidden x 4*hidden");
    for (prad_buf_t o : {dG_next, dG})
        if (int32_t st = same_shape(gates, o, "LSTM step backward")) return st;
    for (prad_buf_t o : {tanh_c, dh_loss, dc_in, dc_prev, dh_scratch})
        if (o != nullptr)
            if (int32_t st = same_shape(c_prev, o, "LSTM step backward")) return st;
    ENQUEUE_LOCK();
    return gates->dtype == PRAD_F64
               ? lstm_step_bwd_t<double>(dG_next, Wh, gates, c_prev, tanh_c, dh_loss, dc_in, dG, dc_prev, dh_scratch)
               : lstm_step_bwd_t<float>(dG_next, Wh, gates, c_prev, tanh_c, dh_loss, dc_in, dG, dc_prev, dh_scratch);
}

// Whole sequences: shape checks shared by both directions.  `gates` is steps*batch x 4*hidden.
static int32_t lstm_sequence_check(prad_buf_t Wh, prad_buf_t gates, int64_t steps, int64_t* batch, int64_t* hidden) {
    if (steps < 1 || gates->depth != 1 || gates->rows % steps != 0 || gates->cols % 4 != 0)
        return fail(PRAD_ERR_ARG, "gates must be steps*batch x 4*hidden");
    *batch = gates->rows / steps;
    *hidden = gates->cols / 4;
    if (Wh->depth != 1 || Wh->rows != *hidden || Wh->cols != 4 * *hidden) return fail(PRAD_ERR_SHAPE, "recurrent weight must be hidden x 4*hidden");
    return PRAD_OK;
}
static int lstm_spin_limit() {
    const char* e = getenv("PRAD_LSTM_SPIN_LIMIT");  // polls of a peer's flag before a workgroup gives up
    const long v = e ? atol(e) : 0;
    if (v < 0) return -1;  // a testing aid: the co-residency probe reports failure without polling
    return v > 0 ? (int)std::min<long>(v, 1L << 30) : (1 << 22);
}
static int32_t expect_rows(prad_buf_t b, int64_t rows, int64_t cols, const char* what) {
    if (b->depth != 1 || b->rows != rows || b->cols != cols) return fail(PRAD_ERR_ARG, "%s must be %lld x %lld", what, (long long)rows, (long long)cols);
    return PRAD_OK;
}

int32_t prad_lstm_sequence_supported(int32_t dtype, int64_t batch, int64_t hidden, int64_t steps) {
    if (!g_ctx.initialized.load()) return 0;
    std::lock_guard<std::mutex> lock(g_ctx.mu);
    return g_ctx.seq_enabled && dtype == PRAD_F32 && lstm_seq_eligible(batch, hidden, steps, g_ctx.compute_units) ? 1 : 0;
}

int32_t prad_lstm_sequence_enable(int32_t on) {
    REQUIRE_INIT();
    ENQUEUE_LOCK();
    g_ctx.seq_enabled = on != 0;
    g_ctx.seq_proven_grid = 0;  // the next sequence call asks the device again
    return PRAD_OK;
}

// A 2-D window of `rows` rows of a buffer, starting at row0 (lives on the caller's stack).
static prad_buf row_window(prad_buf_t b, int64_t row0, int64_t rows) {
    return prad_buf{BUF_MAGIC, b->dtype, 1, rows, b->cols, static_cast<char*>(b->ptr) + (size_t)row0 * b->cols * elem_size(b->dtype), false, 0};
}

// Lock held.  Whether this call may use the sequence kernels: the shape fits, they are on, and the device has been
// seen to hold a grid of this size at once.  The first call for a larger grid than any before asks the device with
// the probe kernel and waits for its answer (once; not inside a recording, where an unproven grid takes the per-step
// path); a probe that gives up turns the sequence kernels off.
static int32_t sequence_kernels_usable(int32_t dtype, int64_t batch, int64_t hidden, int64_t steps, bool* usable) {
    *usable = false;
    if (!g_ctx.seq_enabled || dtype != PRAD_F32 || !lstm_seq_eligible(batch, hidden, steps, g_ctx.compute_units)) return PRAD_OK;
    const int grid = (int)((batch / 16) * (hidden / 16));
    if (grid <= g_ctx.seq_proven_grid) { *usable = true; return PRAD_OK; }
    if (g_ctx.recording) return PRAD_OK;
    if (int32_t st = sync_all()) return st;
    HIP_TRY(launch_lstm_seq_probe(batch, hidden, g_ctx.seq_flags, g_ctx.seq_abort, lstm_spin_limit(), CUR_STREAM), PRAD_ERR_LAUNCH);
    ++g_ctx.stat_stream_syncs;
    HIP_TRY(hipStreamSynchronize(g_ctx.stream), PRAD_ERR_LAUNCH);
    if (*static_cast<volatile unsigned*>(g_ctx.seq_abort) != 0u) {
        *static_cast<volatile unsigned*>(g_ctx.seq_abort) = 0u;
        g_ctx.seq_enabled = false;
        tl_error = "the device does not hold the LSTM sequence kernels' whole grid at once (other work holds compute units): "
                   "prad_lstm_sequence_fwd / _bwd run one launch per time step";
        return PRAD_OK;
    }
    g_ctx.seq_proven_grid = grid;
    g_ctx.seq_groups_local = static_cast<volatile unsigned*>(g_ctx.seq_abort)[1] == 0u;
    static_cast<volatile unsigned*>(g_ctx.seq_abort)[1] = 0u;
    *usable = true;
    return PRAD_OK;
}

extern "C++" {
// The same sequence as `steps` launches each way (lock held): the path of every shape and element type the sequence
// kernels do not take, and of every call once they are off.
template <typename T>
static int32_t lstm_sequence_fwd_steps(prad_buf_t Wh, prad_buf_t G, prad_buf_t C, prad_buf_t Hs, prad_buf_t TC, int64_t steps, int64_t B) {
    for (int64_t t = 0; t < steps; ++t) {
        prad_buf h_prev = row_window(Hs, t * B, B), g = row_window(G, t * B, B), c_prev = row_window(C, t * B, B);
        prad_buf c = row_window(C, (t + 1) * B, B), tc = row_window(TC, t * B, B), h = row_window(Hs, (t + 1) * B, B);
        if (int32_t st = lstm_step_fwd_t<T>(&h_prev, Wh, &g, &c_prev, &c, &tc, &h)) return st;
    }
    return PRAD_OK;
}

template <typename T>
static int32_t lstm_sequence_bwd_steps(prad_buf_t Wh, prad_buf_t gates, prad_buf_t C, prad_buf_t TC, prad_buf_t dHl, prad_buf_t dG,
                                       int64_t steps, int64_t B, int64_t H) {
    const size_t block = (((size_t)B * H * sizeof(T)) + 255) & ~(size_t)255;
    if (g_ctx.seq_step_scratch_bytes < 4 * block) {
        if (g_ctx.recording)
            return fail(PRAD_ERR_RECORDING, "the per-time-step scratch would have to grow during a recording: run the sequence once before recording it");
        void* fresh = nullptr;
        size_t klass = 0;
        if (int32_t st = pool_take(4 * block, &fresh, &klass)) return st;
        if (g_ctx.seq_step_scratch) (void)pool_give(g_ctx.seq_step_scratch, g_ctx.seq_step_scratch_class);
        g_ctx.seq_step_scratch = fresh; g_ctx.seq_step_scratch_bytes = 4 * block; g_ctx.seq_step_scratch_class = klass;
    }
    char* base = static_cast<char*>(g_ctx.seq_step_scratch);
    prad_buf rec[2], dc[2];
    for (int i = 0; i < 2; ++i) {
        rec[i] = prad_buf{BUF_MAGIC, gates->dtype, 1, B, H, base + (size_t)i * block, false, 0};
        dc[i] = prad_buf{BUF_MAGIC, gates->dtype, 1, B, H, base + (size_t)(2 + i) * block, false, 0};
    }
    for (int64_t t = steps - 1; t >= 0; --t) {
        prad_buf g = row_window(gates, t * B, B), c_prev = row_window(C, t * B, B), tc = row_window(TC, t * B, B);
        prad_buf dhl = row_window(dHl, t * B, B), dg = row_window(dG, t * B, B);
        prad_buf* dc_in = &dc[t % 2];
        prad_buf* dc_out = &dc[(t + 1) % 2];
        if (t == steps - 1) {  // the last time step has no recurrent part and no dc arriving
            HIP_TRY(launch_lstm_cell_bwd<T>(static_cast<const T*>(g.ptr), static_cast<const T*>(c_prev.ptr), static_cast<const T*>(tc.ptr),
                                            static_cast<const T*>(dhl.ptr), nullptr, nullptr, static_cast<T*>(dg.ptr),
                                            static_cast<T*>(dc_out->ptr), B, H, CUR_STREAM), PRAD_ERR_LAUNCH);
            continue;
        }
        prad_buf dg_next = row_window(dG, (t + 1) * B, B);
        if (int32_t st = lstm_step_bwd_t<T>(&dg_next, Wh, &g, &c_prev, &tc, &dhl, dc_in, &dg, dc_out, &rec[t % 2])) return st;
    }
    return PRAD_OK;
}
}  // extern "C++"

int32_t prad_lstm_sequence_fwd(prad_buf_t Wh, prad_buf_t G, prad_buf_t C, prad_buf_t Hs, prad_buf_t tanh_c, int64_t steps) {
    REQUIRE_INIT();
    REQUIRE_BUF(Wh); REQUIRE_BUF(G); REQUIRE_BUF(C); REQUIRE_BUF(Hs); REQUIRE_BUF(tanh_c);
    if (int32_t st = same_dtype({Wh, G, C, Hs, tanh_c})) return st;
    int64_t batch = 0, hidden = 0;
    if (int32_t st = lstm_sequence_check(Wh, G, steps, &batch, &hidden)) return st;
    if (int32_t st = expect_rows(C, (steps + 1) * batch, hidden, "C")) return st;
    if (int32_t st = expect_rows(Hs, (steps + 1) * batch, hidden, "Hs")) return st;
    if (int32_t st = expect_rows(tanh_c, steps * batch, hidden, "tanh_c")) return st;
    ENQUEUE_LOCK();
    bool usable = false;
    if (int32_t st = sequence_kernels_usable(G->dtype, batch, hidden, steps, &usable)) return st;
    if (!usable)
        return G->dtype == PRAD_F64 ? lstm_sequence_fwd_steps<double>(Wh, G, C, Hs, tanh_c, steps, batch)
                                    : lstm_sequence_fwd_steps<float>(Wh, G, C, Hs, tanh_c, steps, batch);
    LstmSeqArgs a{};
    a.Wh = F(Wh); a.G = F(G); a.C = F(C); a.Hs = F(Hs); a.TC = F(tanh_c);
    a.flags = g_ctx.seq_flags; a.abort_word = g_ctx.seq_abort;
    a.batch = (int)batch; a.hidden = (int)hidden; a.steps = (int)steps; a.spin_limit = lstm_spin_limit(); a.local = g_ctx.seq_groups_local ? 1 : 0;
    HIP_TRY(launch_lstm_seq(a, false, CUR_STREAM), PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

int32_t prad_lstm_sequence_bwd(prad_buf_t Wh, prad_buf_t gates, prad_buf_t C, prad_buf_t tanh_c, prad_buf_t dh_loss, prad_buf_t dG,
                               int64_t steps) {
    REQUIRE_INIT();
    REQUIRE_BUF(Wh); REQUIRE_BUF(gates); REQUIRE_BUF(C); REQUIRE_BUF(tanh_c); REQUIRE_BUF(dh_loss); REQUIRE_BUF(dG);
    if (int32_t st = same_dtype({Wh, gates, C, tanh_c, dh_loss, dG})) return st;
    int64_t batch = 0, hidden = 0;
    if (int32_t st = lstm_sequence_check(Wh, gates, steps, &batch, &hidden)) return st;
    if (int32_t st = expect_rows(C, (steps + 1) * batch, hidden, "C")) return st;
    if (int32_t st = expect_rows(tanh_c, steps * batch, hidden, "tanh_c")) return st;
    if (int32_t st = expect_rows(dh_loss, steps * batch, hidden, "dh_loss")) return st;
    if (int32_t st = expect_rows(dG, steps * batch, 4 * hidden, "dG")) return st;
    ENQUEUE_LOCK();
    bool usable = false;
    if (int32_t st = sequence_kernels_usable(gates->dtype, batch, hidden, steps, &usable)) return st;
    if (!usable)
        return gates->dtype == PRAD_F64 ? lstm_sequence_bwd_steps<double>(Wh, gates, C, tanh_c, dh_loss, dG, steps, batch, hidden)
                                        : lstm_sequence_bwd_steps<float>(Wh, gates, C, tanh_c, dh_loss, dG, steps, batch, hidden);
    LstmSeqArgs a{};
    a.Wh = F(Wh); a.G = F(gates); a.C = F(C); a.TC = F(tanh_c); a.dHl = F(dh_loss); a.dG = F(dG);
    if (int32_t st = ensure_workspace(lstm_seq_partial_bytes(batch, hidden))) return st;
    a.partial = static_cast<float*>(CUR_WORKSPACE);
    a.flags = g_ctx.seq_flags; a.abort_word = g_ctx.seq_abort;
    a.batch = (int)batch; a.hidden = (int)hidden; a.steps = (int)steps; a.spin_limit = lstm_spin_limit(); a.local = g_ctx.seq_groups_local ? 1 : 0;
    HIP_TRY(launch_lstm_seq(a, true, CUR_STREAM), PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

int32_t prad_window_attention_supported(int32_t dtype, int64_t tokens, int64_t head_dim) {
    return dtype == PRAD_F32 && window_attention_supported(tokens, head_dim) ? 1 : 0;
}

int32_t prad_window_attention_fwd(prad_buf_t QKV, prad_buf_t P, prad_buf_t O, int64_t windows, int64_t heads, int64_t tokens, double scale) {
    REQUIRE_INIT();
    REQUIRE_BUF(QKV); REQUIRE_BUF(P); REQUIRE_BUF(O);
    if (int32_t st = same_dtype({QKV, P, O})) return st;
    if (windows < 1 || heads < 1 || tokens < 1 || QKV->depth != 1 || QKV->rows != windows * tokens || QKV->cols % (3 * heads) != 0)
        return fail(PRAD_ERR_ARG, "QKV must be (windows*tokens) x (3*heads*head_dim)");
    const int64_t head_dim = QKV->cols / (3 * heads);
    if (QKV->dtype != PRAD_F32 || !window_attention_supported(tokens, head_dim))
        return fail(PRAD_ERR_ARG, "the one-launch attention takes float, head dimension 32 and at most 64 tokens per window; ask "
                                  "prad_window_attention_supported first");
    if (int32_t st = expect_rows(P, heads * windows * tokens, tokens, "P")) return st;
    if (int32_t st = expect_rows(O, windows * tokens, heads * head_dim, "O")) return st;
    ENQUEUE_LOCK();
    HIP_TRY(launch_window_attention_fwd(F(QKV), F(P), F(O), windows, heads, tokens, (float)scale, CUR_STREAM), PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

int32_t prad_window_attention_bwd(prad_buf_t QKV, prad_buf_t P, prad_buf_t dO, prad_buf_t dQKV, int64_t windows, int64_t heads, int64_t tokens,
                                  double scale) {
    REQUIRE_INIT();
    REQUIRE_BUF(QKV); REQUIRE_BUF(P); REQUIRE_BUF(dO); REQUIRE_BUF(dQKV);
    if (int32_t st = same_dtype({QKV, P, dO, dQKV})) return st;
    if (windows < 1 || heads < 1 || tokens < 1 || QKV->depth != 1 || QKV->rows != windows * tokens || QKV->cols % (3 * heads) != 0)
        return fail(PRAD_ERR_ARG, "QKV must be (windows*tokens) x (3*heads*head_dim)");
    const int64_t head_dim = QKV->cols / (3 * heads);
    if (QKV->dtype != PRAD_F32 || !window_attention_supported(tokens, head_dim))
        return fail(PRAD_ERR_ARG, "the one-launch attention takes float, head dimension 32 and at most 64 tokens per window; ask "
                                  "prad_window_attention_supported first");
    if (int32_t st = expect_rows(P, heads * windows * tokens, tokens, "P")) return st;
    if (int32_t st = expect_rows(dO, windows * tokens, heads * head_dim, "dO")) return st;
    if (int32_t st = expect_rows(dQKV, windows * tokens, 3 * heads * head_dim, "dQKV")) return st;
    if (dQKV->ptr == QKV->ptr || dQKV->ptr == dO->ptr) return fail(PRAD_ERR_ARG, "dQKV must not alias an input");
    ENQUEUE_LOCK();
    HIP_TRY(launch_window_attention_bwd(F(QKV), F(P), F(dO), F(dQKV), windows, heads, tokens, (float)scale, CUR_STREAM), PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

int32_t prad_buf_view_rows(prad_buf_t parent, int64_t row0, int64_t rows, prad_buf_t* out) {
    REQUIRE_INIT();
    REQUIRE_BUF(parent);
    if (out == nullptr) return fail(PRAD_ERR_ARG, "out is NULL");
    if (parent->depth != 1 || row0 < 0 || rows <= 0 || row0 + rows > parent->rows) return fail(PRAD_ERR_ARG, "row range outside the buffer");
    char* base = static_cast<char*>(parent->ptr) + (size_t)row0 * parent->cols * elem_size(parent->dtype);
    *out = new prad_buf{BUF_MAGIC, parent->dtype, 1, rows, parent->cols, base, false, 0};
    return PRAD_OK;
}

// ---------------------------------------------------------------------------------------------
// Recording.  The stream is captured in thread-local mode and the context remembers which thread records:
// every enqueueing entry point called from another thread while a recording is open returns
// PRAD_ERR_RECORDING instead of slipping its work into the recorded sequence (the reference calls Backward of
// independent operations from pool threads, src/RMAD/OperationNeuralNetworkVisitor.cs:303-306).
int32_t prad_graph_begin(void) {
    REQUIRE_INIT();
    ENQUEUE_LOCK();
    if (g_ctx.recording) return fail(PRAD_ERR_RECORDING, "a launch sequence is already being recorded");
    HIP_TRY(hipStreamBeginCapture(g_ctx.stream, hipStreamCaptureModeThreadLocal), PRAD_ERR_LAUNCH);
    g_ctx.recording = true;
    g_ctx.recorder = std::this_thread::get_id();
    g_recording_adam_count = 0;
    g_recording_failed = false;
    return PRAD_OK;
}

int32_t prad_graph_end(void** graph) {
    REQUIRE_INIT();
    if (graph == nullptr) return fail(PRAD_ERR_ARG, "graph is NULL");
    *graph = nullptr;
    ENQUEUE_LOCK();
    if (!g_ctx.recording) return fail(PRAD_ERR_ARG, "prad_graph_end without prad_graph_begin");
    g_ctx.recording = false;
    hipGraph_t g = nullptr;
    HIP_TRY(hipStreamEndCapture(g_ctx.stream, &g), PRAD_ERR_LAUNCH);
    if (g_recording_failed) {
        (void)hipGraphDestroy(g);
        return fail(PRAD_ERR_LAUNCH, "the recording lost track of an Adam kernel node");
    }
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g);
        return fail(PRAD_ERR_LAUNCH, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    }
    RecordedGraph* rg = new RecordedGraph{GRAPH_MAGIC, g, exec,
                                          std::vector<AdamNode>(g_recording_adam, g_recording_adam + g_recording_adam_count), 0.0, 0.0};
    g_recording_adam_count = 0;
    if (!rg->adam.empty()) {
        rg->base_t = rg->adam[0].t;
        for (const AdamNode& n : rg->adam) rg->base_t = n.t < rg->base_t ? n.t : rg->base_t;
        rg->next_t = rg->base_t;
    }
    ++g_ctx.live_graphs;
    *graph = rg;
    return PRAD_OK;
}

static RecordedGraph* recorded(void* graph) {
    RecordedGraph* rg = static_cast<RecordedGraph*>(graph);
    return (rg != nullptr && rg->magic == GRAPH_MAGIC) ? rg : nullptr;
}

int32_t prad_graph_set_adam_iteration(void* graph, double t) {
    REQUIRE_INIT();
    ENQUEUE_LOCK();
    RecordedGraph* rg = recorded(graph);
    if (rg == nullptr) return fail(PRAD_ERR_BAD_HANDLE, "not a recorded launch sequence");
    if (!(t >= 1.0)) return fail(PRAD_ERR_ARG, "AdamIteration starts at 1");
    rg->next_t = t;
    return PRAD_OK;
}

int32_t prad_graph_launch(void* graph) {
    REQUIRE_INIT();
    ENQUEUE_LOCK();
    NOT_WHILE_RECORDING("launching a recorded sequence");
    RecordedGraph* rg = recorded(graph);
    if (rg == nullptr) return fail(PRAD_ERR_BAD_HANDLE, "not a recorded launch sequence");
    for (AdamNode& n : rg->adam) {
        const double t = rg->next_t + (n.t - rg->base_t);
        if (t == n.applied) continue;
        if (n.dtype == PRAD_F64) {
            double c1, c2;
            bias_correction(n.beta1, n.beta2, t, &c1, &c2);
            HIP_TRY(adam_node_set_bias_correction<double>(rg->exec, n.node, c1, c2), PRAD_ERR_LAUNCH);
        } else {
            float c1, c2;
            bias_correction((float)n.beta1, (float)n.beta2, (float)t, &c1, &c2);
            HIP_TRY(adam_node_set_bias_correction<float>(rg->exec, n.node, c1, c2), PRAD_ERR_LAUNCH);
        }
        n.applied = t;
    }
    HIP_TRY(hipGraphLaunch(rg->exec, g_ctx.stream), PRAD_ERR_LAUNCH);
    rg->next_t += 1.0;
    return PRAD_OK;
}

int32_t prad_graph_destroy(void* graph) {
    REQUIRE_INIT();
    if (graph == nullptr) return PRAD_OK;
    ENQUEUE_LOCK();
    NOT_WHILE_RECORDING("destroying a recorded sequence");
    RecordedGraph* rg = recorded(graph);
    if (rg == nullptr) return fail(PRAD_ERR_BAD_HANDLE, "not a recorded launch sequence");
    if (int32_t st = sync_all()) return st;
    (void)hipGraphExecDestroy(rg->exec);
    (void)hipGraphDestroy(rg->graph);
    rg->magic = 0;
    delete rg;
    if (g_ctx.live_graphs > 0 && --g_ctx.live_graphs == 0) free_retired_workspaces();
    return PRAD_OK;
}

int32_t prad_softmax_cce(prad_buf_t x, prad_buf_t target, prad_buf_t p, prad_buf_t loss, prad_buf_t dp, prad_buf_t dx) {
    REQUIRE_INIT();
    REQUIRE_BUF(x); REQUIRE_BUF(target); REQUIRE_BUF(p); REQUIRE_BUF(dp); REQUIRE_BUF(dx);
    if (loss != nullptr) REQUIRE_BUF(loss);
    if (int32_t st = same_dtype({x, target, p, loss, dp, dx})) return st;
    if (x->depth != 1) return fail(PRAD_ERR_SHAPE, "deep buffer passed to softmax + cross-entropy");
    if (x->rows != target->rows || x->cols != target->cols || target->depth != 1)
        return fail(PRAD_ERR_ARG, "Output and target matrices must have the same dimensions.");
    if (loss != nullptr && (loss->depth != 1 || loss->rows != 1 || loss->cols != 1)) return fail(PRAD_ERR_ARG, "loss must be 1 x 1");
    for (prad_buf_t o : {p, dp, dx})
        if (int32_t st = same_shape(x, o, "softmax + cross-entropy")) return st;
    ENQUEUE_LOCK();
    DISPATCH(x, launch_softmax_cce<double>(D(x), D(target), D(p), D(dp), D(dx), loss ? D(loss) : nullptr, g_ctx.counter, x->rows, x->cols, CUR_STREAM),
             launch_softmax_cce<float>(F(x), F(target), F(p), F(dp), F(dx), loss ? F(loss) : nullptr, g_ctx.counter, x->rows, x->cols, CUR_STREAM));
    return PRAD_OK;
}

// The classifier's output layer with its loss in one launch where the shape allows, otherwise as the three launches it
// stands for (prad_matmul_fwd_fused, prad_softmax_cce, prad_matmul_bias_bwd): same values either way.
int32_t prad_dense_softmax_cce(prad_buf_t A, prad_buf_t W, prad_buf_t bias, prad_buf_t target, prad_buf_t z, prad_buf_t p,
                               prad_buf_t loss, prad_buf_t dp, prad_buf_t dz, prad_buf_t dA, prad_buf_t dW, prad_buf_t dbias,
                               int32_t accumulate_dW, int32_t act, prad_buf_t act_src, double alpha) {
    REQUIRE_INIT();
    REQUIRE_BUF(A); REQUIRE_BUF(W); REQUIRE_BUF(target); REQUIRE_BUF(z); REQUIRE_BUF(p); REQUIRE_BUF(dp); REQUIRE_BUF(dz);
    REQUIRE_BUF(dA); REQUIRE_BUF(dW);
    if (bias != nullptr) REQUIRE_BUF(bias);
    if (loss != nullptr) REQUIRE_BUF(loss);
    if (dbias != nullptr) REQUIRE_BUF(dbias);
    if (act_src != nullptr) REQUIRE_BUF(act_src);
    if (act < PRAD_ACT_NONE || act > PRAD_ACT_AMPLIFIED_SIGMOID) return fail(PRAD_ERR_ARG, "unknown activation %d", act);
    if (act != PRAD_ACT_NONE && act_src == nullptr) return fail(PRAD_ERR_ARG, "an activation's Backward needs the operand it cached");
    if (int32_t st = same_dtype({A, W, bias, target, z, p, loss, dp, dz, dA, dW, dbias, act_src})) return st;
    const bool flat = A->depth == 1 && W->depth == 1 && target->depth == 1 && z->depth == 1 && p->depth == 1 && dp->depth == 1 &&
                      dz->depth == 1 && dA->depth == 1 && dW->depth == 1 && (bias == nullptr || bias->depth == 1) &&
                      (dbias == nullptr || dbias->depth == 1) && (act_src == nullptr || act_src->depth == 1);
    const int64_t B = A->rows, H = A->cols, C = W->cols;
    const bool shapes = flat && W->rows == H && target->rows == B && target->cols == C && z->rows == B && z->cols == C && p->rows == B &&
                        p->cols == C && dp->rows == B && dp->cols == C && dz->rows == B && dz->cols == C && dA->rows == B &&
                        dA->cols == H && dW->rows == H && dW->cols == C && (bias == nullptr || (bias->rows == 1 && bias->cols == C)) &&
                        (dbias == nullptr || (dbias->rows == 1 && dbias->cols == C)) &&
                        (act_src == nullptr || (act_src->rows == B && act_src->cols == H)) &&
                        (loss == nullptr || (loss->rows == 1 && loss->cols == 1));
    ENQUEUE_LOCK();
    // (the one-launch kernel reads the cached operand of later tiles after it has stored earlier ones: an input gradient
    // written over that operand, which the separate launches allow element by element, goes to them)
    const bool in_place = act_src != nullptr && dA->ptr == act_src->ptr;
    const bool one_launch = shapes && !in_place && (A->dtype == PRAD_F64 ? prad::classifier_head_eligible<double>(B, H, C)
                                                                         : prad::classifier_head_eligible<float>(B, H, C));
    if (!one_launch) {  // the separate launches, which also word the complaint about a shape that fits none of them
        Epilogue fwd;
        fwd.bias = bias; fwd.alpha = alpha;
        if (int32_t st = enqueue_gemm(0, 0, A, W, z, 0, fwd, false)) return st;
        if (z->rows != target->rows || z->cols != target->cols || target->depth != 1)
            return fail(PRAD_ERR_ARG, "Output and target matrices must have the same dimensions.");
        if (loss != nullptr && (loss->depth != 1 || loss->rows != 1 || loss->cols != 1)) return fail(PRAD_ERR_ARG, "loss must be 1 x 1");
        for (prad_buf_t o : {p, dp, dz})
            if (int32_t st = same_shape(z, o, "softmax + cross-entropy")) return st;
        DISPATCH(z, launch_softmax_cce<double>(D(z), D(target), D(p), D(dp), D(dz), loss ? D(loss) : nullptr, g_ctx.counter, z->rows, z->cols, CUR_STREAM),
                 launch_softmax_cce<float>(F(z), F(target), F(p), F(dp), F(dz), loss ? F(loss) : nullptr, g_ctx.counter, z->rows, z->cols, CUR_STREAM));
        Epilogue bwd;
        bwd.act_bwd = act; bwd.act_src = act_src; bwd.alpha = alpha;
        return matmul_bwd_locked(dz, A, W, dA, dW, 0, accumulate_dW, bwd, dbias);
    }
#define HEAD_ARGS(T, PTR)                                                                                                   \
    prad::HeadArgs<T> h{};                                                                                                  \
    h.A = PTR(A); h.W = PTR(W); h.bias = bias ? PTR(bias) : nullptr; h.target = PTR(target);                               \
    h.act_src = act_src ? PTR(act_src) : nullptr; h.Z = PTR(z); h.P = PTR(p); h.loss = loss ? PTR(loss) : nullptr;         \
    h.dP = PTR(dp); h.dZ = PTR(dz); h.dA = PTR(dA); h.dW = PTR(dW); h.dbias = dbias ? PTR(dbias) : nullptr;                \
    h.B = (int)B; h.H = (int)H; h.C = (int)C; h.act = act; h.alpha = (T)alpha; h.accumulate_dW = accumulate_dW ? 1 : 0;     \
    HIP_TRY(prad::launch_classifier_head<T>(h, CUR_STREAM), PRAD_ERR_LAUNCH);
    if (A->dtype == PRAD_F64) { HEAD_ARGS(double, D) } else { HEAD_ARGS(float, F) }
#undef HEAD_ARGS
    return PRAD_OK;
}

// ---------------------------------------------------------------------------------------------
int32_t prad_clip_multi(const prad_buf_t* g, int32_t n, double clip_value, double min_value) {
    REQUIRE_INIT();
    if (n < 0 || (n > 0 && g == nullptr)) return fail(PRAD_ERR_ARG, "bad tensor list");
    if (n == 0) return PRAD_OK;
    for (int i = 0; i < n; ++i) {
        REQUIRE_BUF(g[i]);
        if (g[i]->dtype != g[0]->dtype) return fail(PRAD_ERR_DTYPE, "buffers of different element types in one call");
    }
    std::vector<int64_t> sizes((size_t)n);
    for (int i = 0; i < n; ++i) sizes[i] = count(g[i]);
    ENQUEUE_LOCK();
    if (int32_t st = ensure_workspace(clip_workspace_bytes(sizes.data(), n))) return st;
    if (g[0]->dtype == PRAD_F64) {
        std::vector<TensorDesc<double>> d((size_t)n);
        for (int i = 0; i < n; ++i) d[i] = TensorDesc<double>{D(g[i]), nullptr, nullptr, nullptr, sizes[i]};
        HIP_TRY(launch_clip<double>(d.data(), n, CUR_WORKSPACE, clip_value, min_value, CUR_STREAM), PRAD_ERR_LAUNCH);
    } else {
        std::vector<TensorDesc<float>> d((size_t)n);
        for (int i = 0; i < n; ++i) d[i] = TensorDesc<float>{F(g[i]), nullptr, nullptr, nullptr, sizes[i]};
        HIP_TRY(launch_clip<float>(d.data(), n, CUR_WORKSPACE, (float)clip_value, (float)min_value, CUR_STREAM), PRAD_ERR_LAUNCH);
    }
    return PRAD_OK;
}

int32_t prad_clip(prad_buf_t g, double clip_value, double min_value) { return prad_clip_multi(&g, 1, clip_value, min_value); }

// Shared by prad_adam_multi (clip == false) and prad_clip_adam_multi.
static int32_t adam_multi(const prad_buf_t* w, const prad_buf_t* m, const prad_buf_t* v, const prad_buf_t* g, int32_t n, bool clip,
                          double clip_value, double min_value, double lr, double beta1, double beta2, double eps, double t,
                          bool reverse = false) {
    REQUIRE_INIT();
    if (n < 0 || (n > 0 && (w == nullptr || m == nullptr || v == nullptr || g == nullptr))) return fail(PRAD_ERR_ARG, "bad tensor list");
    if (n == 0) return PRAD_OK;
    for (int i = 0; i < n; ++i) {
        REQUIRE_BUF(w[i]); REQUIRE_BUF(m[i]); REQUIRE_BUF(v[i]); REQUIRE_BUF(g[i]);
        for (prad_buf_t o : {w[i], m[i], v[i], g[i]})
            if (o->dtype != w[0]->dtype) return fail(PRAD_ERR_DTYPE, "buffers of different element types in one call");
        for (prad_buf_t o : {m[i], v[i], g[i]})
            if (int32_t st = same_shape(w[i], o, "Adam")) return st;
    }
    std::vector<int64_t> sizes((size_t)n);
    for (int i = 0; i < n; ++i) sizes[i] = count(w[i]);
    ENQUEUE_LOCK();
    if (clip)
        if (int32_t st = ensure_workspace(clip_workspace_bytes(sizes.data(), n))) return st;
    PendingAdam pending{w[0]->dtype, beta1, beta2, t};
    const AdamLaunchObserver observer{note_adam_node, &pending};
    const AdamLaunchObserver* obs = (g_ctx.recording && !reverse) ? &observer : nullptr;
    if (w[0]->dtype == PRAD_F64) {
        double c1, c2;
        bias_correction(beta1, beta2, t, &c1, &c2);
        std::vector<TensorDesc<double>> d((size_t)n);
        for (int i = 0; i < n; ++i) d[i] = TensorDesc<double>{D(g[i]), D(w[i]), D(m[i]), D(v[i]), sizes[i]};
        if (clip)
            HIP_TRY(launch_clip_adam<double>(d.data(), n, CUR_WORKSPACE, clip_value, min_value, lr, beta1, beta2, eps, c1, c2, CUR_STREAM, obs),
                    PRAD_ERR_LAUNCH);
        else
            HIP_TRY(launch_adam<double>(d.data(), n, lr, beta1, beta2, eps, c1, c2, reverse, CUR_STREAM, obs), PRAD_ERR_LAUNCH);
    } else {
        const float b1 = (float)beta1, b2 = (float)beta2;
        float c1, c2;
        bias_correction(b1, b2, (float)t, &c1, &c2);
        std::vector<TensorDesc<float>> d((size_t)n);
        for (int i = 0; i < n; ++i) d[i] = TensorDesc<float>{F(g[i]), F(w[i]), F(m[i]), F(v[i]), sizes[i]};
        if (clip)
            HIP_TRY(launch_clip_adam<float>(d.data(), n, CUR_WORKSPACE, (float)clip_value, (float)min_value, (float)lr, b1, b2,
                                            (float)eps, c1, c2, CUR_STREAM, obs),
                    PRAD_ERR_LAUNCH);
        else
            HIP_TRY(launch_adam<float>(d.data(), n, (float)lr, b1, b2, (float)eps, c1, c2, reverse, CUR_STREAM, obs), PRAD_ERR_LAUNCH);
    }
    return PRAD_OK;
}

// The allocation-free form of prad_clip_adam_multi: no hipMalloc, no hipFree, no host heap.  The chunk moments of the
// clip statistics go to the static device array `scratch` (through the address looked up at prad_init) instead of the
// growable workspace.  Every call on a device shares that array, so calls must not overlap on a device: here they
// cannot, because every call is enqueued on the one library stream.  Nothing in it needs to start at zero (the statistics
// pass writes every slot that the later passes read), so a call after a larger one is not disturbed by what that left.
int32_t prad_clip_adam_multi_noalloc(const prad_buf_t* w, const prad_buf_t* m, const prad_buf_t* v, const prad_buf_t* g, int32_t n,
                                     double clip_value, double min_value, double lr, double beta1, double beta2, double eps,
                                     double t) {
    REQUIRE_INIT();
    constexpr int MAX_TENSORS = 64;
    if (n < 0 || (n > 0 && (w == nullptr || m == nullptr || v == nullptr || g == nullptr))) return fail(PRAD_ERR_ARG, "bad tensor list");
    if (n == 0) return PRAD_OK;
    if (n > MAX_TENSORS) return fail(PRAD_ERR_ARG, "the allocation-free form takes at most %d tensors per call (got %d)", MAX_TENSORS, n);
    int64_t sizes[MAX_TENSORS];
    for (int i = 0; i < n; ++i) {
        REQUIRE_BUF(w[i]); REQUIRE_BUF(m[i]); REQUIRE_BUF(v[i]); REQUIRE_BUF(g[i]);
        for (prad_buf_t o : {w[i], m[i], v[i], g[i]})
            if (o->dtype != w[0]->dtype) return fail(PRAD_ERR_DTYPE, "buffers of different element types in one call");
        for (prad_buf_t o : {m[i], v[i], g[i]})
            if (int32_t st = same_shape(w[i], o, "Adam")) return st;
        sizes[i] = count(w[i]);
    }
    const size_t need = clip_workspace_bytes(sizes, n);
    if (need > STATIC_SCRATCH_BYTES)
        return fail(PRAD_ERR_ARG, "the tensors need %zu bytes of clip statistics, the static scratch holds %zu (about %lld elements in all); "
                    "use prad_clip_adam_multi", need, STATIC_SCRATCH_BYTES, (long long)(STATIC_SCRATCH_BYTES / 24 * 4096));
    ENQUEUE_LOCK();
    void* const ptr = g_scratch_ptr[g_ctx.device];
    if (ptr == nullptr) return fail(PRAD_ERR_NOT_INITIALIZED, "the static scratch has no address on device %d", g_ctx.device);
    PendingAdam pending{w[0]->dtype, beta1, beta2, t};
    const AdamLaunchObserver observer{note_adam_node, &pending};
    const AdamLaunchObserver* obs = g_ctx.recording ? &observer : nullptr;
    if (w[0]->dtype == PRAD_F64) {
        double c1, c2;
        bias_correction(beta1, beta2, t, &c1, &c2);
        TensorDesc<double> d[MAX_TENSORS];
        for (int i = 0; i < n; ++i) d[i] = TensorDesc<double>{D(g[i]), D(w[i]), D(m[i]), D(v[i]), sizes[i]};
        HIP_TRY(launch_clip_adam<double>(d, n, ptr, clip_value, min_value, lr, beta1, beta2, eps, c1, c2, CUR_STREAM, obs), PRAD_ERR_LAUNCH);
    } else {
        const float b1 = (float)beta1, b2 = (float)beta2;
        float c1, c2;
        bias_correction(b1, b2, (float)t, &c1, &c2);
        TensorDesc<float> d[MAX_TENSORS];
        for (int i = 0; i < n; ++i) d[i] = TensorDesc<float>{F(g[i]), F(w[i]), F(m[i]), F(v[i]), sizes[i]};
        HIP_TRY(launch_clip_adam<float>(d, n, ptr, (float)clip_value, (float)min_value, (float)lr, b1, b2, (float)eps, c1, c2,
                                        CUR_STREAM, obs), PRAD_ERR_LAUNCH);
    }
    return PRAD_OK;
}

int32_t prad_adam_multi(const prad_buf_t* w, const prad_buf_t* m, const prad_buf_t* v, const prad_buf_t* g, int32_t n, double lr,
                        double beta1, double beta2, double eps, double t) {
    return adam_multi(w, m, v, g, n, false, 0.0, 0.0, lr, beta1, beta2, eps, t);
}

int32_t prad_adam_revert_multi(const prad_buf_t* w, const prad_buf_t* m, const prad_buf_t* v, const prad_buf_t* g, int32_t n,
                               double lr, double beta1, double beta2, double eps, double t) {
    return adam_multi(w, m, v, g, n, false, 0.0, 0.0, lr, beta1, beta2, eps, t, true);
}

int32_t prad_clip_adam_multi(const prad_buf_t* w, const prad_buf_t* m, const prad_buf_t* v, const prad_buf_t* g, int32_t n,
                             double clip_value, double min_value, double lr, double beta1, double beta2, double eps, double t) {
    return adam_multi(w, m, v, g, n, true, clip_value, min_value, lr, beta1, beta2, eps, t);
}

int32_t prad_adam(prad_buf_t w, prad_buf_t m, prad_buf_t v, prad_buf_t g, double lr, double beta1, double beta2, double eps,
                  double t) {
    return prad_adam_multi(&w, &m, &v, &g, 1, lr, beta1, beta2, eps, t);
}

// ---------------------------------------------------------------------------------------------
int32_t prad_event_create(void** ev) {
    REQUIRE_INIT();
    if (ev == nullptr) return fail(PRAD_ERR_ARG, "ev is NULL");
    hipEvent_t e;
    HIP_TRY(hipEventCreate(&e), PRAD_ERR_ALLOC);
    *ev = e;
    return PRAD_OK;
}
int32_t prad_event_destroy(void* ev) {
    REQUIRE_INIT();
    HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(ev)), PRAD_ERR_ARG);
    return PRAD_OK;
}
int32_t prad_event_record(void* ev) {
    REQUIRE_INIT();
    ENQUEUE_LOCK();
    HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(ev), g_ctx.stream), PRAD_ERR_LAUNCH);
    return PRAD_OK;
}
int32_t prad_event_elapsed_ms(void* start, void* stop, float* ms) {
    REQUIRE_INIT();
    if (ms == nullptr) return fail(PRAD_ERR_ARG, "ms is NULL");
    HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(stop)), PRAD_ERR_LAUNCH);
    HIP_TRY(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)), PRAD_ERR_LAUNCH);
    return PRAD_OK;
}

}  // extern "C"
#pragma GCC visibility pop
