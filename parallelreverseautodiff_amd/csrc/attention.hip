// Windowed self-attention of one block per window and head, one launch forward and one backward (float, head dimension
// 32, up to 64 tokens per window; the backward kernel is described where it stands).  Forward: S = Q . K^T
// (MatrixMultiplyOperation, src/RMAD/MatrixMultiplyOperation.cs:50-86), scaled (MatrixMultiplyScalarOperation),
// P = softmax rows (src/RMAD/SoftmaxOperation.cs:45-110), O = P . V - the node sequence
// of examples/swin/SwinExample/SwinTransformerTools.cs:348-399.  As separate launches the 49 x 49 scores of 3072
// windows x heads go to memory and back twice (two products of K = 32 and 49 at 26 us each and a softmax pass at 25 us,
// all bound by that traffic).  Here one wavefront takes one (window, head): the scores stay in its accumulators and its
// LDS tile, only P - which the backward pass needs - is written, and Q, K, V are read once.
//
//   * Q and K fragments come straight from memory: lane (i, g) of a 16 x 16 x 4 MFMA holds k = 8 g .. 8 g + 7 of its
//     row (two 16-byte loads; MFMA step s multiplies the k's {8 g + s}: a permutation of the sum along k, the same for
//     both operands), so a row's 128 bytes are read whole by four lanes;
//   * the 4 x 4 tiles of S are parked in an LDS tile (pitch 65), lane r < tokens takes row r through the softmax exactly
//     as softmax_fwd_rows_kernel does (scale, maximum, exp, sum in ascending column order, divide), columns past the
//     window become zeros;
//   * P leaves as the contiguous tokens x tokens block it is in memory, and feeds the second product as the A operand
//     from the same tile; V fragments were fetched at the start.
#include "common.h"

#include <cstdlib>

namespace prad {

namespace {

typedef float f4a __attribute__((ext_vector_type(4)));
constexpr int ATT_HD = 32;      // head dimension
constexpr int ATT_PITCH = 65;   // LDS tile pitch (odd: a lane walking its row and 16 lanes reading a column meet no conflicts)
constexpr int ATT_WAVES = 4;

struct AttArgs {
    const float* QKV;  // tokens_total x (3 * heads * 32): [Q | K | V], a head's 32 columns inside each
    float* P;          // [head][window][tokens][tokens]
    float* O;          // tokens_total x (heads * 32)
    int windows, heads, tokens;
    float scale;
};

__device__ __forceinline__ float att_exp(float x) { return __expf(x); }

// The sum of a value over the four lanes (li, 0..3) that share li.
__device__ __forceinline__ float sum_over_g(float v) {
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
// Dot product of two rows' k = 8 g .. 8 g + 7 (the lane's share; sum_over_g completes it).
__device__ __forceinline__ float dot8(const f4a (&a)[2], const f4a (&b)[2]) {
    float d = 0.f;
#pragma unroll
    for (int v = 0; v < 2; ++v)
#pragma unroll
        for (int c = 0; c < 4; ++c) d += a[v][c] * b[v][c];
    return d;
}

// KS: k steps of the product that reduces over the tokens (13 for windows of 49 to 52 tokens, else 16).  FR: windows of
// exactly 49 tokens - three 16 x 16 tiles each way on the matrix cores and the 49th row and column (a fringe that would
// cost seven more tiles of sixteen, all but one row or column of each padding) as dot products on the vector unit.
template <int KS, bool FR>
__global__ void __launch_bounds__(64 * ATT_WAVES, FR ? 3 : 2) window_attention_fwd_kernel(const AttArgs p) {
    constexpr int TX = FR ? 3 : 4;    // 16 x 16 tiles each way on the matrix cores
    constexpr int NC = FR ? 49 : 64;  // columns the softmax walks
    // FR: nothing reaches past row 48 or column 51, and a tile of 49 x 53 lets three workgroups share a compute unit
    // instead of two: the 3072 (window, head) pairs of the 16 x 56 x 56 block are then resident at once, three to a SIMD,
    // instead of a round and a half of two (31 -> 27 us).  The backward kernel needs 220 registers, more than three
    // wavefronts to a SIMD leave each (168): tried with the loads of its last operands moved down, it spilled and ran at
    // 49 us against 46.
    constexpr int ROWS = FR ? 49 : 64, PITCH = FR ? 53 : ATT_PITCH;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int li = lane & 15, g = lane >> 4;
    const int64_t pair = (int64_t)blockIdx.x * ATT_WAVES + wave;  // (window, head), heads innermost
    __shared__ float tiles[ATT_WAVES][ROWS * PITCH];
    if (pair >= (int64_t)p.windows * p.heads) return;
    const int w = (int)(pair / p.heads), h = (int)(pair % p.heads);
    const int wt = FR ? 49 : p.tokens, C = p.heads * ATT_HD, ld = 3 * C;
    float* __restrict__ tile = tiles[wave];
    const float* __restrict__ Q = p.QKV + (int64_t)w * wt * ld + h * ATT_HD;
    const float* __restrict__ K = Q + C;
    const float* __restrict__ V = Q + 2 * C;

    // fragments of Q and K: row 16 x + li (rows past the window: the last row again, never stored - with FR every lane's
    // fragment 3 is row 48), k = 8 g .. 8 g + 7
    f4a qf[4][2], kf[4][2];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        const int row = min(16 * x + li, wt - 1);
#pragma unroll
        for (int v = 0; v < 2; ++v) {
            qf[x][v] = *reinterpret_cast<const f4a*>(Q + (int64_t)row * ld + 8 * g + 4 * v);
            kf[x][v] = *reinterpret_cast<const f4a*>(K + (int64_t)row * ld + 8 * g + 4 * v);
        }
    }
    // fragments of V for the second product: token 4 s + g (clamped: P is zero there), column 16 y + li
    float vf[KS][2];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int tok = min(4 * s + g, wt - 1);
#pragma unroll
        for (int y = 0; y < 2; ++y) vf[s][y] = V[(int64_t)tok * ld + 16 * y + li];
    }

    // S = Q . K^T
    f4a acc[TX][TX];
#pragma unroll
    for (int x = 0; x < TX; ++x)
#pragma unroll
        for (int y = 0; y < TX; ++y) acc[x][y] = f4a{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
        for (int x = 0; x < TX; ++x)
#pragma unroll
            for (int y = 0; y < TX; ++y) acc[x][y] = __builtin_amdgcn_mfma_f32_16x16x4f32(qf[x][s >> 2][s & 3], kf[y][s >> 2][s & 3], acc[x][y], 0, 0, 0);
    if constexpr (FR) {  // row 48 and column 48 of S
        float fr[3], fc[3];
#pragma unroll
        for (int y = 0; y < 3; ++y) {
            fr[y] = sum_over_g(dot8(qf[3], kf[y]));  // S[48][16 y + li]
            fc[y] = sum_over_g(dot8(qf[y], kf[3]));  // S[16 y + li][48]
        }
        const float corner = sum_over_g(dot8(qf[3], kf[3]));
        if (g == 0) {
#pragma unroll
            for (int y = 0; y < 3; ++y) {
                tile[48 * PITCH + 16 * y + li] = fr[y];
                tile[(16 * y + li) * PITCH + 48] = fc[y];
            }
            if (li == 0) tile[48 * PITCH + 48] = corner;
        }
    }
#pragma unroll
    for (int x = 0; x < TX; ++x)
#pragma unroll
        for (int y = 0; y < TX; ++y)
#pragma unroll
            for (int r = 0; r < 4; ++r) tile[(16 * x + 4 * g + r) * PITCH + 16 * y + li] = acc[x][y][r];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // softmax of row `lane` (the arithmetic of softmax_fwd_rows_kernel); the columns past the window become zeros
    // (with FR the rows past the window hold whatever the tile held: nothing reads them)
    if (!FR || lane < ROWS) {
        float* __restrict__ row = tile + lane * PITCH;
        float v[NC];
#pragma unroll
        for (int j = 0; j < NC; ++j) v[j] = j < wt ? row[j] * p.scale : -INFINITY;
        float m = v[0];
#pragma unroll
        for (int j = 1; j < NC; ++j) m = fmaxf(m, v[j]);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < NC; ++j) {
            v[j] = j < wt ? att_exp(v[j] - m) : 0.f;
            sum = sum + v[j];
        }
        // one division per row, a multiplication per element (within an ulp of the quotient): float MFMAs do not overlap
        // with vector instructions on this chip (measured), so the ten instructions of a division, forty-nine times a
        // row, were time the products of the other wavefronts on this SIMD did not get
        const float inv = 1.0f / sum;
#pragma unroll
        for (int j = 0; j < NC; ++j) row[j] = j < wt ? v[j] * inv : 0.f;
#pragma unroll
        for (int j = NC; j < 4 * KS; ++j) row[j] = 0.f;  // (FR: the k steps of the second product reach column 51)
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // P leaves as one contiguous block
    {
        float* __restrict__ dst = p.P + ((int64_t)h * p.windows + w) * wt * wt;
        int r = lane / wt, c = lane % wt;  // element lane + 64 i
        const int dr = 64 / wt, dc = 64 % wt;
        for (int e = lane; e < wt * wt; e += 64) {
            dst[e] = tile[r * PITCH + c];
            r += dr; c += dc;
            if (c >= wt) { c -= wt; ++r; }
        }
    }

    // O = P . V: rows 16 x + li of P from the tile, k = token
    f4a out[TX][2];
#pragma unroll
    for (int x = 0; x < TX; ++x)
#pragma unroll
        for (int y = 0; y < 2; ++y) out[x][y] = f4a{0.f, 0.f, 0.f, 0.f};
    // (all KS steps whatever the window: P is zero past it, and a branch per step would send the accumulators through copies)
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        float a[TX];
#pragma unroll
        for (int x = 0; x < TX; ++x) a[x] = tile[(16 * x + li) * PITCH + 4 * s + g];
#pragma unroll
        for (int x = 0; x < TX; ++x)
#pragma unroll
            for (int y = 0; y < 2; ++y) out[x][y] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[x], vf[s][y], out[x][y], 0, 0, 0);
    }
    float* __restrict__ O = p.O + (int64_t)w * wt * C + h * ATT_HD;
    if constexpr (FR) {  // row 48 of O
        float o2[2] = {0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const float pv = tile[48 * PITCH + 4 * s + g];
#pragma unroll
            for (int y = 0; y < 2; ++y) o2[y] += pv * vf[s][y];
        }
#pragma unroll
        for (int y = 0; y < 2; ++y) {
            o2[y] = sum_over_g(o2[y]);
            if (g == 0) O[(int64_t)48 * C + 16 * y + li] = o2[y];
        }
    }
#pragma unroll
    for (int x = 0; x < TX; ++x)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = 16 * x + 4 * g + r;
            if (row < wt) {
#pragma unroll
                for (int y = 0; y < 2; ++y) O[(int64_t)row * C + 16 * y + li] = out[x][y][r];
            }
        }
}

// Backward of the same nodes for one (window, head) per wavefront: with dO the gradient of O,
//   dP = dO . V^T ;  dV = P^T . dO ;  dS = P (.) (dP - rowsum(dP (.) P)) * scale  (SoftmaxOperation.Backward followed by the
//   scalar product's, src/RMAD/SoftmaxOperation.cs:75-110) ;  dQ = dS . K ;  dK = dS^T . Q
// - five launches and four trips of the 49 x 49 blocks through memory when taken one by one.  P comes into the
// wavefront's LDS tile once (zeros past the window), serves dV as the A operand read across, and the softmax's backward
// in the accumulators' own layout; dS then takes the tile's place for the last two products.  KS = k steps of the three
// products whose reduction runs over the tokens (13 for windows of 49 to 52 tokens, else 16).
struct AttBwdArgs {
    const float* QKV; const float* P; const float* dO; float* dQKV;
    int windows, heads, tokens;
    float scale;
};

template <int KS, bool FR>
__global__ void __launch_bounds__(64 * ATT_WAVES, 2) window_attention_bwd_kernel(const AttBwdArgs p) {
    constexpr int TX = FR ? 3 : 4;  // 16 x 16 tiles each way on the matrix cores (FR: windows of 49 tokens, as in the forward kernel)
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int li = lane & 15, g = lane >> 4;
    const int64_t pair = (int64_t)blockIdx.x * ATT_WAVES + wave;
    __shared__ float tiles[ATT_WAVES][64 * ATT_PITCH];
    if (pair >= (int64_t)p.windows * p.heads) return;
    const int w = (int)(pair / p.heads), h = (int)(pair % p.heads);
    const int wt = FR ? 49 : p.tokens, C = p.heads * ATT_HD, ld = 3 * C;
    float* __restrict__ tile = tiles[wave];
    const float* __restrict__ Q = p.QKV + (int64_t)w * wt * ld + h * ATT_HD;
    const float* __restrict__ K = Q + C;
    const float* __restrict__ V = Q + 2 * C;
    const float* __restrict__ dO = p.dO + (int64_t)w * wt * C + h * ATT_HD;
    const float* __restrict__ P = p.P + ((int64_t)h * p.windows + w) * wt * wt;

    // token-major fragments of an operand whose rows are tokens: element [token 4 s + g][16 y + li] (tokens past the window: the last one;
    // they meet zeros of P or dS)
    auto token_frags = [&](const float* __restrict__ base, int64_t pitch, float (&f)[KS][2]) {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const int tok = min(4 * s + g, wt - 1);
#pragma unroll
            for (int y = 0; y < 2; ++y) f[s][y] = base[(int64_t)tok * pitch + 16 * y + li];
        }
    };
    // every operand that comes from memory is asked for before the first product, the ones used last, last
    f4a af[4][2], bf[4][2];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        const int row = min(16 * x + li, wt - 1);
#pragma unroll
        for (int v = 0; v < 2; ++v) {
            af[x][v] = *reinterpret_cast<const f4a*>(dO + (int64_t)row * C + 8 * g + 4 * v);
            bf[x][v] = *reinterpret_cast<const f4a*>(V + (int64_t)row * ld + 8 * g + 4 * v);
        }
    }
    // P -> tile, zeros past the window; sixteen loads in flight per lane
    for (int e = lane; e < 64 * ATT_PITCH / 4; e += 64) reinterpret_cast<f4a*>(tile)[e] = f4a{0.f, 0.f, 0.f, 0.f};
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    {
        int r = lane / wt, c = lane % wt;
        const int dr = 64 / wt, dc = 64 % wt, n = wt * wt;
        for (int e0 = lane; e0 < n; e0 += 64 * 16) {
            float v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) v[u] = P[min(e0 + 64 * u, n - 1)];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                if (e0 + 64 * u < n) tile[r * ATT_PITCH + c] = v[u];
                r += dr; c += dc;
                if (c >= wt) { c -= wt; ++r; }
            }
        }
    }
    float dof[KS][2], kf[KS][2], qf[KS][2];
    token_frags(dO, C, dof);
    token_frags(K, ld, kf);
    token_frags(Q, ld, qf);
    // dP = dO . V^T: rows of dO and V as k-contiguous fragments (k = 8 g .. 8 g + 7, as in the forward kernel)
    f4a acc[TX][TX];
#pragma unroll
    for (int x = 0; x < TX; ++x)
#pragma unroll
        for (int y = 0; y < TX; ++y) acc[x][y] = f4a{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
        for (int x = 0; x < TX; ++x)
#pragma unroll
            for (int y = 0; y < TX; ++y) acc[x][y] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[x][s >> 2][s & 3], bf[y][s >> 2][s & 3], acc[x][y], 0, 0, 0);
    // FR: dP[48][16 y + li], dP[16 x + li][48] and dP[48][48], each on all four lanes that share li
    float dpr[3] = {0.f, 0.f, 0.f}, dpc[3] = {0.f, 0.f, 0.f}, dpk = 0.f;
    if constexpr (FR) {
#pragma unroll
        for (int y = 0; y < 3; ++y) {
            dpr[y] = sum_over_g(dot8(af[3], bf[y]));
            dpc[y] = sum_over_g(dot8(af[y], bf[3]));
        }
        dpk = sum_over_g(dot8(af[3], bf[3]));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    auto store_block = [&](float* __restrict__ dst, const f4a (&o)[TX][2]) {  // rows = tokens, 32 columns of this head
#pragma unroll
        for (int x = 0; x < TX; ++x)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = 16 * x + 4 * g + r;
                if (row < wt) {
#pragma unroll
                    for (int y = 0; y < 2; ++y) dst[(int64_t)row * ld + 16 * y + li] = o[x][y][r];
                }
            }
    };
    // One product that reduces over the tokens: A fragments from the tile (element (m, k) at m * pitch_m + k * pitch_k),
    // B the token-major fragments f; FR: output row 48 on the vector unit, from the tile's row or column 48.
    auto token_product = [&](int pitch_m, int pitch_k, const float (&f)[KS][2], float* __restrict__ dst) {
        f4a o[TX][2];
#pragma unroll
        for (int x = 0; x < TX; ++x)
#pragma unroll
            for (int y = 0; y < 2; ++y) o[x][y] = f4a{0.f, 0.f, 0.f, 0.f};
        float o2[2] = {0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            float a[TX];
#pragma unroll
            for (int x = 0; x < TX; ++x) a[x] = tile[(16 * x + li) * pitch_m + (4 * s + g) * pitch_k];
#pragma unroll
            for (int x = 0; x < TX; ++x)
#pragma unroll
                for (int y = 0; y < 2; ++y) o[x][y] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[x], f[s][y], o[x][y], 0, 0, 0);
            if constexpr (FR) {
                const float a48 = tile[48 * pitch_m + (4 * s + g) * pitch_k];
#pragma unroll
                for (int y = 0; y < 2; ++y) o2[y] += a48 * f[s][y];
            }
        }
        if constexpr (FR) {
#pragma unroll
            for (int y = 0; y < 2; ++y) {
                o2[y] = sum_over_g(o2[y]);
                if (g == 0) dst[(int64_t)48 * ld + 16 * y + li] = o2[y];
            }
        }
        store_block(dst, o);
    };
    float* __restrict__ dQ = p.dQKV + (int64_t)w * wt * ld + h * ATT_HD;

    // dV = P^T . dO: A = P read across (row j of P^T = column j of P), k = token i
    token_product(1, ATT_PITCH, dof, dQ + 2 * C);
    // dS = P (.) (dP - rowsum(dP (.) P)) * scale in the accumulators' layout: acc[x][y][r] is (row 16 x + 4 g + r, column 16 y + li)
    float dsc[TX][4];  // FR: dS[16 x + 4 g + r][48]
#pragma unroll
    for (int x = 0; x < TX; ++x)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float pv[TX], dot = 0.f;
#pragma unroll
            for (int y = 0; y < TX; ++y) {
                pv[y] = tile[(16 * x + 4 * g + r) * ATT_PITCH + 16 * y + li];
                dot += acc[x][y][r] * pv[y];
            }
#pragma unroll
            for (int m = 1; m < 16; m <<= 1) dot += __shfl_xor(dot, m, 64);  // over the 16 lanes that share the row
            if constexpr (FR) {  // the row's 49th column: dP from the lane whose li is this row's, P from the tile
                const float dp48 = __shfl(dpc[x], 4 * g + r, 64), p48 = tile[(16 * x + 4 * g + r) * ATT_PITCH + 48];
                dot += dp48 * p48;
                dsc[x][r] = (p48 * (dp48 - dot)) * p.scale;
            }
#pragma unroll
            for (int y = 0; y < TX; ++y) acc[x][y][r] = (pv[y] * (acc[x][y][r] - dot)) * p.scale;
        }
    float ds48[3] = {0.f, 0.f, 0.f}, dsk = 0.f;  // FR: dS[48][16 y + li], dS[48][48]
    if constexpr (FR) {
        float p48[3], dot = 0.f;
#pragma unroll
        for (int y = 0; y < 3; ++y) {
            p48[y] = tile[48 * ATT_PITCH + 16 * y + li];
            dot += dpr[y] * p48[y];
        }
#pragma unroll
        for (int m = 1; m < 16; m <<= 1) dot += __shfl_xor(dot, m, 64);
        const float pk = tile[48 * ATT_PITCH + 48];
        dot += dpk * pk;
#pragma unroll
        for (int y = 0; y < 3; ++y) ds48[y] = (p48[y] * (dpr[y] - dot)) * p.scale;
        dsk = (pk * (dpk - dot)) * p.scale;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();  // every lane has read its part of P
#pragma unroll
    for (int x = 0; x < TX; ++x)
#pragma unroll
        for (int y = 0; y < TX; ++y)
#pragma unroll
            for (int r = 0; r < 4; ++r) tile[(16 * x + 4 * g + r) * ATT_PITCH + 16 * y + li] = acc[x][y][r];
    if constexpr (FR) {
        if (li == 0) {
#pragma unroll
            for (int x = 0; x < TX; ++x)
#pragma unroll
                for (int r = 0; r < 4; ++r) tile[(16 * x + 4 * g + r) * ATT_PITCH + 48] = dsc[x][r];
        }
        if (g == 0) {
#pragma unroll
            for (int y = 0; y < 3; ++y) tile[48 * ATT_PITCH + 16 * y + li] = ds48[y];
            if (li == 0) tile[48 * ATT_PITCH + 48] = dsk;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // dQ = dS . K (A = dS rows) and dK = dS^T . Q (A = dS read across)
    token_product(ATT_PITCH, 1, kf, dQ);
    token_product(1, ATT_PITCH, qf, dQ + C);
}

}  // namespace

bool window_attention_supported(int64_t tokens, int64_t head_dim) {
    static const bool enabled = [] { const char* e = getenv("PRAD_ATTENTION_FUSED"); return !(e && e[0] == '0'); }();  // tuning aid
    return enabled && head_dim == ATT_HD && tokens >= 1 && tokens <= 64;
}

hipError_t launch_window_attention_fwd(const float* QKV, float* P, float* O, int64_t windows, int64_t heads, int64_t tokens, float scale,
                                       hipStream_t stream) {
    if (!window_attention_supported(tokens, ATT_HD) || reinterpret_cast<uintptr_t>(QKV) % 16 != 0) return hipErrorNotSupported;
    AttArgs a{QKV, P, O, (int)windows, (int)heads, (int)tokens, scale};
    const int64_t pairs = windows * heads;
    const dim3 grid((unsigned)((pairs + ATT_WAVES - 1) / ATT_WAVES)), block(64 * ATT_WAVES);
    if (tokens == 49) hipLaunchKernelGGL((window_attention_fwd_kernel<13, true>), grid, block, 0, stream, a);
    else if (tokens > 48 && tokens <= 52) hipLaunchKernelGGL((window_attention_fwd_kernel<13, false>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((window_attention_fwd_kernel<16, false>), grid, block, 0, stream, a);
    return hipGetLastError();
}

hipError_t launch_window_attention_bwd(const float* QKV, const float* P, const float* dO, float* dQKV, int64_t windows, int64_t heads,
                                       int64_t tokens, float scale, hipStream_t stream) {
    if (!window_attention_supported(tokens, ATT_HD) || reinterpret_cast<uintptr_t>(QKV) % 16 != 0 || reinterpret_cast<uintptr_t>(dO) % 16 != 0)
        return hipErrorNotSupported;
    AttBwdArgs a{QKV, P, dO, dQKV, (int)windows, (int)heads, (int)tokens, scale};
    const int64_t pairs = windows * heads;
    const dim3 grid((unsigned)((pairs + ATT_WAVES - 1) / ATT_WAVES)), block(64 * ATT_WAVES);
    if (tokens == 49) hipLaunchKernelGGL((window_attention_bwd_kernel<13, true>), grid, block, 0, stream, a);
    else if (tokens > 48 && tokens <= 52) hipLaunchKernelGGL((window_attention_bwd_kernel<13, false>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((window_attention_bwd_kernel<16, false>), grid, block, 0, stream, a);
    return hipGetLastError();
}

}  // namespace prad
