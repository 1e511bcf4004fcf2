// LSTM cell arithmetic around the fused 4-gate matrix product.  The reference wires an LSTM step from
// separate operation nodes - SigmoidOperation (src/RMAD/SigmoidOperation.cs:46-84), TanhOperation
// (src/RMAD/TanhOperation.cs:42-79), HadamardProductOperation (src/RMAD/HadamardProductOperation.cs:50-118)
// and MatrixAddOperation (src/RMAD/MatrixAddOperation.cs:29-66), see
// examples/lstm/.../architecture/SelfAttentionMultiLayerLSTMArchitectureAmplified.json - each a
// scalar loop over batch x hidden.  Here the ten of them per time step are one pass over the
// pre-activations in each direction, with every formula kept as those operations write it.
//
// Layout: G is batch x 4*hidden, gate blocks [i | f | g | o] side by side in each row.
#include "common.h"

namespace prad {

template <typename T>
__global__ void __launch_bounds__(256) lstm_cell_fwd_kernel(T* __restrict__ G, const T* __restrict__ c_prev, T* __restrict__ c,
                                                            T* __restrict__ tanh_c, T* __restrict__ h, int64_t rows, int64_t hidden) {
    const int64_t n = rows * hidden;
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * 256) {
        const int64_t r = idx / hidden, j = idx % hidden;
        T* __restrict__ g = G + r * 4 * hidden;
        const T i_ = act_forward<T>(ACT_SIGMOID, g[j], (T)0);
        const T f_ = act_forward<T>(ACT_SIGMOID, g[hidden + j], (T)0);
        const T g_ = act_forward<T>(ACT_TANH, g[2 * hidden + j], (T)0);
        const T o_ = act_forward<T>(ACT_SIGMOID, g[3 * hidden + j], (T)0);
        g[j] = i_; g[hidden + j] = f_; g[2 * hidden + j] = g_; g[3 * hidden + j] = o_;  // activated gates, kept for backward
        const T cn = (f_ * c_prev[idx]) + (i_ * g_);  // Hadamard, Hadamard, MatrixAdd
        const T tc = act_forward<T>(ACT_TANH, cn, (T)0);
        c[idx] = cn;
        tanh_c[idx] = tc;
        h[idx] = o_ * tc;
    }
}

// dh = dh_a + dh_b (loss path + recurrent path; dh_b may be null), dc_in may be null (last step).
template <typename T>
__global__ void __launch_bounds__(256) lstm_cell_bwd_kernel(const T* __restrict__ gates, const T* __restrict__ c_prev,
                                                            const T* __restrict__ tanh_c, const T* __restrict__ dh_a,
                                                            const T* __restrict__ dh_b, const T* __restrict__ dc_in,
                                                            T* __restrict__ dG, T* __restrict__ dc_prev, int64_t rows, int64_t hidden) {
    const int64_t n = rows * hidden;
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * 256) {
        const int64_t r = idx / hidden, j = idx % hidden;
        const T* __restrict__ g = gates + r * 4 * hidden;
        T* __restrict__ dg = dG + r * 4 * hidden;
        const T i_ = g[j], f_ = g[hidden + j], g_ = g[2 * hidden + j], o_ = g[3 * hidden + j];
        const T tc = tanh_c[idx];
        T dh = dh_a[idx];
        if (dh_b != nullptr) dh = dh + dh_b[idx];
        const T d_o = dh * tc;                                              // Hadamard backward (h = o . tanh c)
        T dc = (dh * o_) * act_derivative<T>(ACT_TANH, tc, (T)0);           // Tanh backward on tanh(c)
        if (dc_in != nullptr) dc = dc + dc_in[idx];                         // gradients of c_t from step t+1 add up
        const T d_i = dc * g_, d_g = dc * i_, d_f = dc * c_prev[idx];       // Hadamard backward twice
        dc_prev[idx] = dc * f_;
        dg[j] = d_i * act_derivative<T>(ACT_SIGMOID, i_, (T)0);
        dg[hidden + j] = d_f * act_derivative<T>(ACT_SIGMOID, f_, (T)0);
        dg[2 * hidden + j] = d_g * act_derivative<T>(ACT_TANH, g_, (T)0);
        dg[3 * hidden + j] = d_o * act_derivative<T>(ACT_SIGMOID, o_, (T)0);
    }
}

template <typename T>
hipError_t launch_lstm_cell_fwd(T* G, const T* c_prev, T* c, T* tanh_c, T* h, int64_t rows, int64_t hidden, hipStream_t s) {
    const int64_t n = rows * hidden;
    if (n <= 0) return hipSuccess;
    int64_t blocks = (n + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL((lstm_cell_fwd_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s, G, c_prev, c, tanh_c, h, rows, hidden);
    return hipGetLastError();
}
template <typename T>
hipError_t launch_lstm_cell_bwd(const T* gates, const T* c_prev, const T* tanh_c, const T* dh_a, const T* dh_b, const T* dc_in,
                                T* dG, T* dc_prev, int64_t rows, int64_t hidden, hipStream_t s) {
    const int64_t n = rows * hidden;
    if (n <= 0) return hipSuccess;
    int64_t blocks = (n + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL((lstm_cell_bwd_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s, gates, c_prev, tanh_c, dh_a, dh_b, dc_in,
                       dG, dc_prev, rows, hidden);
    return hipGetLastError();
}

#define INSTANTIATE(T)                                                                                               \
    template hipError_t launch_lstm_cell_fwd<T>(T*, const T*, T*, T*, T*, int64_t, int64_t, hipStream_t);            \
    template hipError_t launch_lstm_cell_bwd<T>(const T*, const T*, const T*, const T*, const T*, const T*, T*, T*,  \
                                                int64_t, int64_t, hipStream_t);
INSTANTIATE(double)
INSTANTIATE(float)

}  // namespace prad
