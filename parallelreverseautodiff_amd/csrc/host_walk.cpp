// A compiled caller of the C ABI: the feed-forward training step walked operation by operation, the way the
// reference's own loop drives its operation objects (forward walk over the node list with a fresh output Matrix per
// node, examples/feedforward/ParallelReverseAutoDiff.FeedForwardExample/FeedForwardNeuralNetwork.cs:212-251; loss;
// backward walk with every node's results added into its gradient destinations, src/RMAD/OperationNeuralNetworkVisitor.cs:198-215
// and src/RMAD/OperationBase.cs:273-304; GradientClearer, GradientClipper.Clip, AdamOptimizer.Optimize over the layers).
// It stands where the reference's C# classes would stand once they bind libprad_hip.so through P/Invoke: nothing but
// calls declared in include/prad_hip.h, one kernel per operation, no fused entry point and no recorded sequence.
// libprad_hostwalk.so (host code only, linked against libprad_hip.so) exports one function, which the benchmark and a
// test call: it measures what the boundary costs a compiled caller, without an interpreter between the calls.
#include "../../include/prad_hip.h"

#include <chrono>
#include <cstring>
#include <vector>

namespace {

struct Failure { int32_t status; };
inline void ok(int32_t status) { if (status != PRAD_OK) throw Failure{status}; }

// An operation's output slot: a fresh buffer per call, the one before it released (it goes back to the library's pool).
struct Slot {
    prad_buf_t buf = nullptr;
    prad_buf_t fresh(int32_t dtype, int64_t rows, int64_t cols) {
        prad_buf_t next = nullptr;
        ok(prad_buf_alloc_output(dtype, 1, rows, cols, &next));
        if (buf != nullptr) ok(prad_buf_free(buf));
        buf = next;
        return buf;
    }
    void release() { if (buf != nullptr) { (void)prad_buf_free(buf); buf = nullptr; } }
};

struct Layer {
    prad_buf_t W = nullptr, b = nullptr, dW = nullptr, db = nullptr, mW = nullptr, vW = nullptr, mb = nullptr, vb = nullptr;
    Slot product, biased, activated;   // MatrixMultiply, MatrixAddBroadcasting, LeakyReLU (or Softmax for the last layer)
    prad_buf_t input = nullptr;        // what MatrixMultiplyOperation.Forward retained (not owned)
};

}  // namespace

extern "C" __attribute__((visibility("default")))
int32_t prad_hostwalk_mlp(int32_t dtype, int32_t batch, int32_t nlayers, const int64_t* sizes, const void* const* weights,
                          const void* X, const void* T, int32_t steps, int32_t warmup, double alpha, double clip_value,
                          double min_clip, double lr, double beta1, double beta2, double eps, double* wall_ms_per_step,
                          double* loss_out, void* const* weights_out) {
    std::vector<Layer> net((size_t)nlayers);
    prad_buf_t x = nullptr, t = nullptr;
    Slot loss, dP;
    std::vector<prad_buf_t> temporaries;  // backward results, released once consumed
    int32_t status = PRAD_OK;
    try {
        ok(prad_buf_alloc(dtype, batch, sizes[0], &x));
        ok(prad_buf_alloc(dtype, batch, sizes[nlayers], &t));
        ok(prad_buf_upload(x, X, sizes[0]));
        ok(prad_buf_upload(t, T, sizes[nlayers]));
        for (int l = 0; l < nlayers; ++l) {
            Layer& L = net[(size_t)l];
            const int64_t in = sizes[l], out = sizes[l + 1];
            for (prad_buf_t* w : {&L.W, &L.dW, &L.mW, &L.vW}) ok(prad_buf_alloc(dtype, in, out, w));
            for (prad_buf_t* v : {&L.b, &L.db, &L.mb, &L.vb}) ok(prad_buf_alloc(dtype, 1, out, v));
            ok(prad_buf_upload(L.W, weights[l], out));
        }
        std::vector<prad_buf_t> w, m, v, g;
        for (Layer& L : net) {
            w.push_back(L.W); w.push_back(L.b);
            m.push_back(L.mW); m.push_back(L.mb);
            v.push_back(L.vW); v.push_back(L.vb);
            g.push_back(L.dW); g.push_back(L.db);
        }
        auto temporary = [&](int64_t rows, int64_t cols) {
            prad_buf_t b = nullptr;
            ok(prad_buf_alloc_output(dtype, 1, rows, cols, &b));
            temporaries.push_back(b);
            return b;
        };
        auto step = [&](int iteration) {
            ok(prad_zero_multi(g.data(), (int32_t)g.size()));                                    // GradientClearer.Clear
            prad_buf_t value = x;
            for (int l = 0; l < nlayers; ++l) {                                                  // forward walk
                Layer& L = net[(size_t)l];
                const int64_t out = sizes[l + 1];
                L.input = value;
                ok(prad_matmul_fwd(value, L.W, L.product.fresh(dtype, batch, out)));
                ok(prad_add_broadcast_fwd(L.product.buf, L.b, L.biased.fresh(dtype, batch, out)));
                if (l + 1 < nlayers) ok(prad_act_fwd(PRAD_ACT_LEAKYRELU, L.biased.buf, L.activated.fresh(dtype, batch, out), alpha));
                else ok(prad_softmax_fwd(L.biased.buf, L.activated.fresh(dtype, batch, out)));
                value = L.activated.buf;
            }
            ok(prad_cce_fwd(value, t, loss.fresh(dtype, 1, 1)));                                  // loss and its gradient
            ok(prad_cce_bwd(value, t, dP.fresh(dtype, batch, sizes[nlayers])));
            prad_buf_t grad = dP.buf;
            for (int l = nlayers - 1; l >= 0; --l) {                                             // backward walk
                Layer& L = net[(size_t)l];
                const int64_t in = sizes[l], out = sizes[l + 1];
                prad_buf_t dx = temporary(batch, out);
                if (l + 1 < nlayers) ok(prad_act_bwd(PRAD_ACT_LEAKYRELU, L.biased.buf, grad, dx, alpha));
                else ok(prad_softmax_bwd(L.activated.buf, grad, dx));
                grad = dx;
                prad_buf_t dbias = temporary(1, out);                                            // MatrixAddBroadcasting: [dOutput itself, dBias]
                ok(prad_add_broadcast_bwd_bias(grad, dbias));
                ok(prad_accumulate(L.db, dbias));
                prad_buf_t dA = temporary(batch, in), dWt = temporary(in, out);                  // MatrixMultiply: [dA, dB], always both
                ok(prad_matmul_bwd(grad, L.input, L.W, dA, dWt, 0, 0));
                ok(prad_accumulate(L.dW, dWt));
                grad = dA;
            }
            for (prad_buf_t b : temporaries) ok(prad_buf_free(b));
            temporaries.clear();
            ok(prad_clip_multi(g.data(), (int32_t)g.size(), clip_value, min_clip));              // GradientClipper.Clip
            ok(prad_adam_multi(w.data(), m.data(), v.data(), g.data(), (int32_t)w.size(), lr, beta1, beta2, eps, (double)iteration));
        };
        int iteration = 0;
        for (int i = 0; i < warmup; ++i) step(++iteration);
        ok(prad_stream_sync());
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < steps; ++i) step(++iteration);
        ok(prad_stream_sync());
        const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        if (wall_ms_per_step != nullptr) *wall_ms_per_step = steps > 0 ? ms / steps : 0.0;
        if (loss_out != nullptr && loss.buf != nullptr) {
            if (dtype == PRAD_F64) ok(prad_buf_download(loss.buf, loss_out, 1));
            else { float f = 0.f; ok(prad_buf_download(loss.buf, &f, 1)); *loss_out = (double)f; }
        }
        if (weights_out != nullptr)
            for (int l = 0; l < nlayers; ++l) ok(prad_buf_download(net[(size_t)l].W, weights_out[l], sizes[l + 1]));
    } catch (const Failure& f) {
        status = f.status;
    }
    for (prad_buf_t b : temporaries) (void)prad_buf_free(b);
    loss.release(); dP.release();
    for (Layer& L : net) {
        L.product.release(); L.biased.release(); L.activated.release();
        for (prad_buf_t b : {L.W, L.b, L.dW, L.db, L.mW, L.vW, L.mb, L.vb}) if (b != nullptr) (void)prad_buf_free(b);
    }
    if (x != nullptr) (void)prad_buf_free(x);
    if (t != nullptr) (void)prad_buf_free(t);
    return status;
}
