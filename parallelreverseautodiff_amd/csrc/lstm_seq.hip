// A whole LSTM sequence in one launch each way (float): the recurrent product h_{t-1} . W_h of every time step
// with the cell arithmetic, forward, and dh_t = dG_{t+1} . W_h^T with the cell's backward, in reverse.  The reference
// unrolls a sequence into one MatrixMultiplyOperation (src/RMAD/MatrixMultiplyOperation.cs:50-126) plus Sigmoid / Tanh /
// HadamardProduct / MatrixAdd nodes per time step (src/RMAD/ComputationGraph.cs:808-849); run as one launch per time step
// and direction, the recurrence costs what 2 x T dependent launches cost (9 to 11 us each for 0.27 GFLOP), about 17 % of
// the matrix cores.  Here the time loop is inside the kernel:
//
//   * the batch rows are cut into groups of 16 and the hidden units into blocks of 16; workgroup (r, c) owns rows
//     [16 r, 16 r + 16) x units [16 c, 16 c + 16) for the whole sequence, one workgroup per compute unit;
//   * its slice of W_h - the 64 columns [gate q][16 c .. 16 c + 16) forward, the same 64 columns as rows of W_h^T
//     backward - is 128 KB for hidden = 512 and lives in the registers of its four wavefronts (128 per lane) for
//     the whole sequence: W_h is read from memory once per launch instead of once per time step;
//   * a time step depends on the other workgroups of its row group only (rows are independent): forward each
//     workgroup publishes its 16 x 16 block of h_t and gathers the group's whole 16 x hidden block; backward each
//     multiplies its own 16 x 64 block of dG_{t+1} by its rows of W_h^T into a partial dh for all hidden units,
//     publishes it cut by consumer, and every workgroup adds the partial blocks meant for it in producer order
//     (deterministic).  The exchange is per-producer flags, no atomics and no device-wide barrier: a producer writes
//     its block with device-scope stores, waits for them (vmcnt(0)), then writes its flag; a consumer polls the flags
//     of its group (one lane per producer) and then reads with device-scope loads.  One exchange round trip was
//     measured at 3 us among 32 workgroups, against 9 to 11 us for a launch per step.
//
// Every wait is bounded: a workgroup that polls `spin_limit` times in vain (the grid is not co-resident, or
// a peer gave up) writes the abort word, which the host checks at its next synchronisation, and leaves; every
// other workgroup then leaves at its next wait.  The arithmetic per element is that of lstm_cell_fwd_kernel /
// lstm_cell_bwd_kernel, statement for statement; only the order of the sums along K differs from the per-step kernels.
#include "common.h"

#include <algorithm>
#include <cstdlib>

namespace prad {

typedef float f4v __attribute__((ext_vector_type(4)));

constexpr int SEQ_THREADS = 256;
constexpr int SEQ_MAX_J = 32;  // hidden / 16 at most: hidden <= 512 (the slice of W_h must fit the registers)
// More than half a compute unit's LDS per workgroup, so that no two workgroups of a grid share a compute unit while
// another stands empty: the step time is that of the slowest workgroup.
constexpr int SEQ_LDS_FLOATS = 21 * 1024;
constexpr int SEQ_STAGE = 16 * (16 * SEQ_MAX_J / 4) / SEQ_THREADS;  // 16-byte vectors of a 16 x hidden block per thread, at most
static_assert(16 * SEQ_MAX_J / 4 * 17 * 4 <= SEQ_LDS_FLOATS, "the staged block (rows padded to 17 vectors) must fit");

// Keeps an LDS array the kernel does not otherwise need in the allocation.
__device__ __forceinline__ void keep_allocated(float* lds) { asm volatile("" : : "v"(lds) : "memory"); }


// 16 bytes at `base + byte_offset` with a device-scope load; `base` must be uniform over the wavefront (it becomes the
// buffer descriptor; a descriptor that differs per lane would be executed lane by lane).
__device__ __forceinline__ f4v coherent_load4(const float* base, int byte_offset) {
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, -1, 0x00020000);
    return __builtin_bit_cast(f4v, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, 16 /* sc1: device scope */));
}
__device__ __forceinline__ float coherent_load(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void coherent_store(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// All of this wavefront's stores so far are acknowledged (a device-scope store is written through).
__device__ __forceinline__ void wait_for_stores() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
}

// Waits until the `blocks` flags at `flags` have all reached `want` (called by every thread of the workgroup; the
// first wavefront polls, one lane per flag).  Returns false - for the whole workgroup - when it gave up.
__device__ __forceinline__ bool wait_for_group(const unsigned* flags, int blocks, unsigned want, unsigned* abort_word, int spin_limit,
                                               int* all_arrived /* LDS */) {
    if (threadIdx.x < 64) {
        bool done = (int)threadIdx.x >= blocks;
        int spins = 0;
        bool ok = true;
        while (true) {
            if (!done) done = __hip_atomic_load(flags + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= want;
            if (__all(done)) break;
            ++spins;
            if (spins > spin_limit || ((spins & 1023) == 0 && __hip_atomic_load(abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0u)) {
                ok = false;
                break;
            }
        }
        if (threadIdx.x == 0) {
            if (!ok) __hip_atomic_store(abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            *all_arrived = ok ? 1 : 0;
        }
    }
    __syncthreads();
    return *all_arrived != 0;
}

// ---- exchange inside one XCD ---------------------------------------------------------------------------------------
// When the workgroups of a row group all sit on one XCD (group index = blockIdx % groups with groups a multiple of the
// eight XCDs, workgroups being dealt to the XCDs round robin from wherever the dispatch before left off), they share that
// XCD's L2: a plain store lands there and a
// load that bypasses the compute unit's own cache (device scope) reads it back from there, with no write-through to
// memory, no acknowledgement to wait for and no flag.  The data itself says that it has arrived: the destination is
// filled with a bit pattern no result can have (a NaN that arithmetic never produces; a NaN result is stored as the
// canonical one) and a consumer reads until the pattern is gone.  Measured on 32 workgroups exchanging 16 x 512 floats
// per step: 1.6 us per step against 2.3 us with write-through stores, acknowledgement, flag and flag poll.  (The forward
// kernel with plain stores but the flags kept was measured too: 1037 us per training step of the 64-step layer against
// 1021 us with the values announcing themselves and 1099 us with device-scope stores.)
constexpr unsigned SEQ_SENTINEL = 0xFFFFFFFFu;
__device__ __forceinline__ bool arrived(const f4v v) {
    // (each element through a plain float first: a bit cast applied directly to a vector element reads element 0.)
    // The sentinel is the largest unsigned value: none of the four is it exactly when their maximum is not.
    const float a = v[0], b = v[1], c = v[2], d = v[3];
    const unsigned m = max(max(__float_as_uint(a), __float_as_uint(b)), max(__float_as_uint(c), __float_as_uint(d)));
    return m != SEQ_SENTINEL;
}
__device__ __forceinline__ float never_the_sentinel(float x) { return x != x ? __builtin_bit_cast(float, 0x7FC00000u) : x; }
// The XCD this wavefront runs on (hardware register XCC_ID).
__device__ __forceinline__ unsigned xcd_of_this_wave() {
    unsigned v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 0xFu;
}

// The cell's sigmoid and tanh for the sequence kernel: float arithmetic on the hardware exponential and reciprocal
// (within 3e-7 of the double-precision evaluation the per-step kernels round to float) - five transcendental functions
// per element sit on every time step's critical path, and in double they cost half a microsecond of it.
__device__ __forceinline__ float seq_sigmoid(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }
__device__ __forceinline__ float seq_tanh(float x) {
    const float t = __expf(-2.0f * fabsf(x));
    return copysignf((1.0f - t) * __builtin_amdgcn_rcpf(1.0f + t), x);
}

// ---- forward ----------------------------------------------------------------------------------------------------
template <bool LOCAL>
__global__ void __launch_bounds__(SEQ_THREADS, 1) lstm_seq_fwd_kernel(const LstmSeqArgs p) {
    const int H = p.hidden, B = p.batch, NJ = H / 16, groups = B / 16, blocks = H / 16;
    const int r = blockIdx.x % groups, c = blockIdx.x / groups;
    const int tid = threadIdx.x, lane = tid & 63, q = tid >> 6;  // wavefront q multiplies for gate q
    const int n = lane & 15, g = lane >> 4;
    const int row = tid >> 4, u = tid & 15;                      // the element this thread finishes: (row, unit u)
    __shared__ __attribute__((aligned(16))) float hblock[SEQ_LDS_FLOATS];  // h_{t-1} rows of the group, as MFMA fragments (16 x hidden used)
    __shared__ float exch[4 * 16 * 16];                              // the four gates' products, [gate][row][unit]
    __shared__ int all_arrived;
    __shared__ int gave_up;
    keep_allocated(hblock);
    const unsigned my_xcd = LOCAL ? xcd_of_this_wave() + 1u : 0u;
    if (LOCAL) {
        // every workgroup of the group must share this XCD's L2 (see above): each says where it runs (a device-scope
        // store into its flag), and before the first exchange every workgroup compares the group's answers with its own
        if (tid == 0) {
            gave_up = 0;
            __hip_atomic_store(p.flags + r * blocks + c, my_xcd, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
    }

    // W_h slice of this wavefront in registers: vector j of lane (n, g) = W_h[16 j + 4 g + i][q H + 16 c + n], i = 0..3
    // (buffer loads: the lane's part of the address is one register for all 128 of them, the (j, i) part a scalar;
    // with per-lane 64-bit addresses every load costs a dozen dependent instructions of a wavefront that runs alone)
    f4v w[SEQ_MAX_J];
    {
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.Wh), 0, -1, 0x00020000);
        const int lane_off = 4 * (4 * g * 4 * H + q * H + 16 * c + n);
#pragma unroll
        for (int j = 0; j < SEQ_MAX_J; ++j) {
            if (j < NJ) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    w[j][i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, lane_off, 4 * (16 * j + i) * 4 * H, 0));
            }
        }
    }
    const int64_t own = (int64_t)(16 * r + row) * H + 16 * c + u;  // offset of (row, u) inside a batch x hidden block
    float c_prev = p.C[own];
    // the vectors of the group's 16 x hidden block this thread stages every step: where from (bytes) and where to (floats)
    int stage_src[SEQ_STAGE], stage_dst[SEQ_STAGE];
#pragma unroll
    for (int e = 0; e < SEQ_STAGE; ++e) {
        const int v = e * SEQ_THREADS + tid, vecs_per_row = H / 4;
        const int m = v / vecs_per_row, kv = v % vecs_per_row;  // kv = 4 j + g'
        stage_src[e] = v < 16 * vecs_per_row ? (m * H + kv * 4) * 4 : -1;
        stage_dst[e] = (kv * 17 + m) * 4;
    }
    unsigned* my_flag = p.flags + r * blocks + c;
    const unsigned* group_flags = p.flags + r * blocks;

    for (int t = 0; t < p.steps; ++t) {
        // pre-activations of this thread's four gates (x_t . W_x + b, from the launch before this one)
        float* grow = p.G + (int64_t)(t * B + 16 * r + row) * 4 * H + 16 * c + u;
        float pre[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) pre[k] = grow[k * H];
        if (!LOCAL && t > 0 && !wait_for_group(group_flags, blocks, (unsigned)t, p.abort_word, p.spin_limit, &all_arrived)) return;
        // h_{t-1} rows of the group -> LDS in fragment order: vector (j, g') of row m = h[m][16 j + 4 g' .. + 3] at slot (4 j + g') * 17 + m
        const float* hsrc = p.Hs + (int64_t)(t * B + 16 * r) * H;
        f4v hv[SEQ_STAGE];
        if (LOCAL) {
            if (t == 1 && tid < 64) {
                bool same = true;
                if (tid < blocks) {
                    unsigned other = 0u;
                    for (int spins = 0; other == 0u && spins <= p.spin_limit; ++spins)
                        other = __hip_atomic_load(p.flags + r * blocks + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    same = other == my_xcd;
                }
                if (!__all(same)) {
                    if (tid == 0) __hip_atomic_store(p.abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    gave_up = 1;
                }
            }
            // read until every vector holds results (block 0, the initial state, is there from the start)
            unsigned pending = 0u;
#pragma unroll
            for (int e = 0; e < SEQ_STAGE; ++e)
                if (stage_src[e] >= 0) pending |= 1u << e;
            int spins = 0;
            while (pending) {
#pragma unroll
                for (int e = 0; e < SEQ_STAGE; ++e)
                    if (pending & (1u << e)) hv[e] = coherent_load4(hsrc, stage_src[e]);
#pragma unroll
                for (int e = 0; e < SEQ_STAGE; ++e)
                    if ((pending & (1u << e)) && arrived(hv[e])) pending &= ~(1u << e);
                if (pending && (++spins > p.spin_limit ||
                                ((spins & 255) == 0 && __hip_atomic_load(p.abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0u))) {
                    __hip_atomic_store(p.abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    gave_up = 1;
                    break;
                }
            }
        } else {
#pragma unroll
            for (int e = 0; e < SEQ_STAGE; ++e)
                if (stage_src[e] >= 0) hv[e] = coherent_load4(hsrc, stage_src[e]);
        }
#pragma unroll
        for (int e = 0; e < SEQ_STAGE; ++e)
            if (stage_src[e] >= 0) *reinterpret_cast<f4v*>(&hblock[stage_dst[e]]) = hv[e];
        __syncthreads();
        if (LOCAL && gave_up) return;
        f4v acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < SEQ_MAX_J; j += 2) {
            if (j < NJ) {
                const f4v a0 = *reinterpret_cast<const f4v*>(&hblock[((4 * j + g) * 17 + n) * 4]);
                const f4v a1 = *reinterpret_cast<const f4v*>(&hblock[((4 * (j + 1) + g) * 17 + n) * 4]);
#pragma unroll
                for (int i = 0; i < 4; ++i) acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[i], w[j][i], acc0, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; ++i) acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a1[i], w[j + 1][i], acc1, 0, 0, 0);
            }
        }
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) exch[(q * 16 + 4 * g + rr) * 16 + n] = acc0[rr] + acc1[rr];
        __syncthreads();
        // the cell, as lstm_cell_fwd_kernel writes it
        const float i_ = seq_sigmoid(pre[0] + exch[(0 * 16 + row) * 16 + u]);
        const float f_ = seq_sigmoid(pre[1] + exch[(1 * 16 + row) * 16 + u]);
        const float g_ = seq_tanh(pre[2] + exch[(2 * 16 + row) * 16 + u]);
        const float o_ = seq_sigmoid(pre[3] + exch[(3 * 16 + row) * 16 + u]);
        grow[0] = i_; grow[H] = f_; grow[2 * H] = g_; grow[3 * H] = o_;
        const float cn = (f_ * c_prev) + (i_ * g_);
        const float tc = seq_tanh(cn);
        const int64_t blk = (int64_t)B * H;
        p.C[(t + 1) * blk + own] = cn;
        p.TC[t * blk + own] = tc;
        c_prev = cn;
        if (LOCAL) {
            // a plain store into the XCD's L2; the two barriers of the next step keep hblock and exch in order
            p.Hs[(t + 1) * blk + own] = never_the_sentinel(o_ * tc);
            continue;
        }
        coherent_store(p.Hs + (t + 1) * blk + own, o_ * tc);
        wait_for_stores();
        __syncthreads();  // every wavefront's h is in memory; also: hblock and exch are free again
        if (tid == 0) __hip_atomic_store(my_flag, (unsigned)(t + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---- backward ---------------------------------------------------------------------------------------------------
// LOCAL: the group's workgroups share one XCD's L2 (see "exchange inside one XCD"), so the partial blocks are stored
// plainly - they land in that L2 and are acknowledged from there instead of being written through to memory - and the
// flags order the steps as before.  (Values that announce themselves, as in the forward kernel, were measured slower
// here: every thread would poll 32 scattered words and put the pattern back into each, 64 KB of extra stores per
// workgroup and step.)
template <bool LOCAL>
__global__ void __launch_bounds__(SEQ_THREADS, 1) lstm_seq_bwd_kernel(const LstmSeqArgs p) {
    const int H = p.hidden, B = p.batch, groups = B / 16, blocks = H / 16;
    const int r = blockIdx.x % groups, c = blockIdx.x / groups;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int row = tid >> 4, u = tid & 15;
    __shared__ __attribute__((aligned(16))) float dgblock[SEQ_LDS_FLOATS];  // this workgroup's dG block as fragments: vector (q, g', m) (16 x 64 used)
    keep_allocated(dgblock);
    __shared__ int all_arrived;
    __shared__ int elsewhere;
    unsigned* xcd_words = p.flags + groups * blocks;  // where each workgroup runs: the words after the progress flags
    const unsigned my_xcd = LOCAL ? xcd_of_this_wave() + 1u : 0u;
    if (LOCAL && tid == 0) {
        elsewhere = 0;
        __hip_atomic_store(xcd_words + r * blocks + c, my_xcd, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // Rows of W_h^T for this workgroup's 64 gate columns, spread over the wavefronts by output unit: wavefront wv
    // produces partial dh for units [tile * 16, tile * 16 + 16), tile = wv + 4 y (y < blocks / 4); vector (y, q) of lane
    // (n, g) = W_h[16 tile + n][q H + 16 c + 4 g + i], i = 0..3.
    constexpr int MAX_Y = SEQ_MAX_J / 4;
    const int NY = blocks / 4;
    f4v w[MAX_Y][4];
#pragma unroll
    for (int y = 0; y < MAX_Y; ++y) {
        if (y < NY) {
            const int unit = 16 * (wv + 4 * y) + n;
#pragma unroll
            for (int qq = 0; qq < 4; ++qq) w[y][qq] = *reinterpret_cast<const f4v*>(p.Wh + (int64_t)unit * 4 * H + qq * H + 16 * c + 4 * g);
        }
    }
    const int64_t own = (int64_t)(16 * r + row) * H + 16 * c + u;
    const int64_t blk = (int64_t)B * H;
    unsigned* my_flag = p.flags + r * blocks + c;
    const unsigned* group_flags = p.flags + r * blocks;
    float dc_next = 0.f;  // gradient of c_t arriving from step t + 1
    float rec = 0.f;      // recurrent part of dh_t: sum over producers of their partial products

    // what the cell's backward of one time step reads, loaded one step ahead (before the wait for the peers)
    struct StepInputs { float i_, f_, g_, o_, tc, dhl, cp; };
    auto load_step = [&](int t) {
        const float* grow = p.G + (int64_t)(t * B + 16 * r + row) * 4 * H + 16 * c + u;
        return StepInputs{grow[0], grow[H], grow[2 * H], grow[3 * H], p.TC[t * blk + own], p.dHl[t * blk + own], p.C[t * blk + own]};
    };
    StepInputs in = load_step(p.steps - 1);

    for (int t = p.steps - 1, s = 0; t >= 0; --t, ++s) {
        const float i_ = in.i_, f_ = in.f_, g_ = in.g_, o_ = in.o_, tc = in.tc, dhl = in.dhl, cp = in.cp;
        // the cell's backward, as lstm_cell_bwd_kernel writes it (the last time step has no recurrent part and no dc_in)
        const float dh = s == 0 ? dhl : dhl + rec;
        const float d_o = dh * tc;
        float dc = (dh * o_) * act_derivative<float>(ACT_TANH, tc, 0.f);
        if (s > 0) dc = dc + dc_next;
        const float d_i = dc * g_, d_g = dc * i_, d_f = dc * cp;
        dc_next = dc * f_;
        float dz[4];
        dz[0] = d_i * act_derivative<float>(ACT_SIGMOID, i_, 0.f);
        dz[1] = d_f * act_derivative<float>(ACT_SIGMOID, f_, 0.f);
        dz[2] = d_g * act_derivative<float>(ACT_TANH, g_, 0.f);
        dz[3] = d_o * act_derivative<float>(ACT_SIGMOID, o_, 0.f);
        float* dgrow = p.dG + (int64_t)(t * B + 16 * r + row) * 4 * H + 16 * c + u;
#pragma unroll
        for (int k = 0; k < 4; ++k) dgrow[k * H] = dz[k];
        if (t == 0) break;
        // this block of dG as the A operand: k = 16 q + u; lane (m, g') reads vector (q, g') = k in [16 q + 4 g', + 4)
#pragma unroll
        for (int k = 0; k < 4; ++k) dgblock[((k * 4 + (u >> 2)) * 16 + row) * 4 + (u & 3)] = dz[k];
        __syncthreads();
        f4v a[4];
#pragma unroll
        for (int qq = 0; qq < 4; ++qq) a[qq] = *reinterpret_cast<const f4v*>(&dgblock[((qq * 4 + g) * 16 + n) * 4]);
        // partial dh_{t-1}[rows][units of tile] = dG block . (W_h rows of the tile)^T, K = 64
        float* pbase = p.partial + (int64_t)(s & 1) * groups * blocks * blocks * 256;
#pragma unroll
        for (int y = 0; y < MAX_Y; ++y) {
            if (y < NY) {
                f4v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int qq = 0; qq < 4; ++qq)
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[qq][i], w[y][qq][i], acc, 0, 0, 0);
                // consumer = the workgroup that owns the tile's units; blocks are laid out [group][consumer][producer][row][unit]
                float* dst = pbase + ((int64_t)((r * blocks + (wv + 4 * y)) * blocks + c) * 16) * 16;
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    if (LOCAL) dst[(4 * g + rr) * 16 + n] = acc[rr];  // a plain store into the XCD's L2
                    else coherent_store(dst + (4 * g + rr) * 16 + n, acc[rr]);
                }
            }
        }
        wait_for_stores();
        __syncthreads();  // (also: dgblock is free again)
        if (tid == 0) __hip_atomic_store(my_flag, (unsigned)(s + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        in = load_step(t - 1);
        if (LOCAL && s == 0 && tid < 64) {  // the group's workgroups all run on this XCD (checked once, before the first exchange)
            bool same = true;
            if (tid < blocks) {
                unsigned other = 0u;
                for (int spins = 0; other == 0u && spins <= p.spin_limit; ++spins)
                    other = __hip_atomic_load(xcd_words + r * blocks + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                same = other == my_xcd;
            }
            if (!__all(same) && tid == 0) {
                __hip_atomic_store(p.abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);  // (the peers leave at their next wait)
                elsewhere = 1;
            }
        }
        if (!wait_for_group(group_flags, blocks, (unsigned)(s + 1), p.abort_word, p.spin_limit, &all_arrived)) return;
        if (LOCAL && elsewhere) return;
        // the blocks meant for this workgroup, added in producer order
        const float* src = pbase + ((int64_t)(r * blocks + c) * blocks * 16) * 16 + row * 16 + u;
        float part[SEQ_MAX_J];
#pragma unroll
        for (int pr = 0; pr < SEQ_MAX_J; ++pr)
            if (pr < blocks) part[pr] = coherent_load(src + pr * 256);
        rec = 0.f;
#pragma unroll
        for (int pr = 0; pr < SEQ_MAX_J; ++pr)
            if (pr < blocks) rec = rec + part[pr];
    }
}

// ---- co-residency probe -------------------------------------------------------------------------------------------
// The sequence kernels need every workgroup of a row group on the device at the same time.  Whether the device can
// hold the grid right now (it cannot when another process or a compute-unit mask takes compute units away) is asked
// once, with a kernel of the same grid, workgroup size and LDS footprint that does nothing but the roll call: every
// workgroup raises its flag and waits, bounded, for the flags of its row group.  Nothing is written but the flags.
__global__ void __launch_bounds__(SEQ_THREADS, 1) lstm_seq_probe_kernel(unsigned* flags, unsigned* abort_word, int spin_limit, int groups,
                                                                       int blocks) {
    __shared__ __attribute__((aligned(16))) float footprint[SEQ_LDS_FLOATS];
    __shared__ int all_arrived;
    keep_allocated(footprint);
    const int r = blockIdx.x % groups, c = blockIdx.x / groups;
    if (spin_limit < 0) {  // forced from the host (tests of the fallback): report failure, wait for nobody
        if (threadIdx.x == 0) __hip_atomic_store(abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        return;
    }
    // the flag value says where the workgroup runs (XCD + 1): the roll call also tells whether each row group sits on
    // one XCD, which decides how the sequence kernels exchange (abort_word[1] is raised if one does not)
    const unsigned mine = xcd_of_this_wave() + 1u;
    if (threadIdx.x == 0) __hip_atomic_store(flags + r * blocks + c, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (!wait_for_group(flags + r * blocks, blocks, 1u, abort_word, spin_limit, &all_arrived)) return;
    if (threadIdx.x < 64) {
        const bool same = (int)threadIdx.x >= blocks ||
                          __hip_atomic_load(flags + r * blocks + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == mine;
        if (!__all(same) && threadIdx.x == 0) __hip_atomic_store(abort_word + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

hipError_t launch_lstm_seq_probe(int64_t batch, int64_t hidden, unsigned* flags, unsigned* abort_word, int spin_limit, hipStream_t s) {
    const int groups = (int)(batch / 16), blocks = (int)(hidden / 16);
    const unsigned grid = (unsigned)(groups * blocks);
    hipError_t e = launch_fill_zero<float>(reinterpret_cast<float*>(flags), grid, s);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(lstm_seq_probe_kernel, dim3(grid), dim3(SEQ_THREADS), 0, s, flags, abort_word, spin_limit, groups, blocks);
    return hipGetLastError();
}

// Shapes the sequence kernels take: float, hidden a multiple of 64 up to 512 (the slice of W_h in registers, the
// backward tiles four wavefronts wide), batch a multiple of 16, one workgroup per compute unit for the whole grid.
bool lstm_seq_eligible(int64_t batch, int64_t hidden, int64_t steps, int compute_units) {
    if (steps < 1 || batch < 16 || batch % 16 != 0 || hidden < 64 || hidden % 64 != 0 || hidden > 16 * SEQ_MAX_J) return false;
    return (batch / 16) * (hidden / 16) <= compute_units;
}
size_t lstm_seq_partial_bytes(int64_t batch, int64_t hidden) {
    return (size_t)2 * (batch / 16) * (hidden / 16) * (hidden / 16) * 256 * sizeof(float);
}

// Fills n floats (a multiple of four, 16-byte aligned) with the bit pattern that means "not written yet".
__global__ void __launch_bounds__(256) seq_sentinel_fill_kernel(f4v* __restrict__ dst, int64_t nvec, unsigned* __restrict__ flags, int nflags) {
    if (blockIdx.x == 0)
        for (int i = threadIdx.x; i < nflags; i += 256) flags[i] = 0u;
    const f4v s = {__builtin_bit_cast(float, SEQ_SENTINEL), __builtin_bit_cast(float, SEQ_SENTINEL), __builtin_bit_cast(float, SEQ_SENTINEL),
                   __builtin_bit_cast(float, SEQ_SENTINEL)};
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) __builtin_nontemporal_store(s, dst + i);
}
// (the same launch zeroes the workgroups' flags)
static hipError_t fill_sentinel(float* dst, int64_t n, unsigned* flags, int nflags, hipStream_t s) {
    const int64_t nvec = n / 4;
    const unsigned blocks = (unsigned)std::min<int64_t>((nvec + 255) / 256, 4096);
    hipLaunchKernelGGL(seq_sentinel_fill_kernel, dim3(blocks), dim3(256), 0, s, reinterpret_cast<f4v*>(dst), nvec, flags, nflags);
    return hipGetLastError();
}

// Whether the row groups of this shape each sit on one XCD (see "exchange inside one XCD"): the group index is
// blockIdx % groups, the XCD blockIdx % 8.  PRAD_LSTM_LOCAL=0 keeps the device-scope exchange (a tuning aid).
bool lstm_seq_local(int64_t batch) {
    static const bool enabled = [] { const char* e = getenv("PRAD_LSTM_LOCAL"); return !(e && e[0] == '0'); }();
    return enabled && (batch / 16) % 8 == 0;
}

hipError_t launch_lstm_seq(const LstmSeqArgs& a, bool backward, hipStream_t s) {
    const unsigned grid = (unsigned)((a.batch / 16) * (a.hidden / 16));
    const bool local = a.local != 0 && lstm_seq_local(a.batch);
    if (!backward && local) {
        // every h_t block that the launch will write starts as "not written yet"
        hipError_t e = fill_sentinel(a.Hs + (int64_t)a.batch * a.hidden, (int64_t)a.steps * a.batch * a.hidden, a.flags, (int)grid, s);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(lstm_seq_fwd_kernel<true>, dim3(grid), dim3(SEQ_THREADS), 0, s, a);
        return hipGetLastError();
    }
    hipError_t e = launch_fill_zero<float>(reinterpret_cast<float*>(a.flags), 2 * grid, s);  // unsigned zero == float zero bits
    if (e != hipSuccess) return e;
    if (backward && local) hipLaunchKernelGGL(lstm_seq_bwd_kernel<true>, dim3(grid), dim3(SEQ_THREADS), 0, s, a);
    else if (backward) hipLaunchKernelGGL(lstm_seq_bwd_kernel<false>, dim3(grid), dim3(SEQ_THREADS), 0, s, a);
    else hipLaunchKernelGGL(lstm_seq_fwd_kernel<false>, dim3(grid), dim3(SEQ_THREADS), 0, s, a);
    return hipGetLastError();
}

}  // namespace prad
