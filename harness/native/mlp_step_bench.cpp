// BASELINE config[4] from a compiled host: the MLP training step (batch 256, 784-512-512-10,
// softmax cross-entropy, backward, Adam) issued through include/zenu_hip.hpp, GEMMs on rocBLAS.
// Same op sequence as tests/mlp_step.py (which cites the reference's files for every line):
//   ops   -- the sequence ZeNu's autograd issues, one library call per Matrix-level op
//   fused -- the same step through the fused entry points
//   lean  -- fused, and the GEMMs take their transposed operands as views (rocBLAS transpose flags)
//            instead of the contiguous copies that ZeNu's autograd `transpose` makes
//            (zenu-autograd/src/functions/transpose.rs:26-33); bias gradients go into
//            uninitialised buffers (sum_to writes every element)
// Prints one line per measurement: "<variant> <what> <value>".
//
//   mlp_step_bench [--inputs file] [--steps K] [--warmup W] [--dump-loss N]
// `file` holds raw little-endian f32: x[256*784], t[256*10], W1[512*784], b1[512], W2[512*512],
// b2[512], W3[10*512], b3[10]; without it the inputs are synthetic (xorshift, same shapes).
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include <rocblas/rocblas.h>

#include "zenu_hip.hpp"

using namespace zenu_hip;
typedef Matrix<float> M;

static const int kBatch = 256;
static const int kLayers[3][2] = {{784, 512}, {512, 512}, {512, 10}};

static rocblas_handle g_blas;

// row-major C[m,n] = A[m,k] B[k,n] through column-major rocBLAS: C^T = B^T A^T
static M gemm(const M &a, const M &b)
{
    const int m = (int)a.shape()[0], k = (int)a.shape()[1], n = (int)b.shape()[1];
    M out = M::alloc({m, n});
    const float alpha = 1.f, beta = 0.f;
    if (rocblas_sgemm(g_blas, rocblas_operation_none, rocblas_operation_none, n, m, k, &alpha, b.as_ptr(), n, a.as_ptr(), k,
                      &beta, out.as_ptr(), n) != rocblas_status_success) {
        std::printf("rocblas_sgemm failed\n");
        std::exit(1);
    }
    return out;
}

// row-major C[m,n] = op(A) op(B), A and B stored row-major with leading dimensions lda, ldb
static M gemm_rm(bool ta, bool tb, int m, int n, int k, const M &a, int lda, const M &b, int ldb)
{
    M out = M::alloc({m, n});
    const float alpha = 1.f, beta = 0.f;
    if (rocblas_sgemm(g_blas, tb ? rocblas_operation_transpose : rocblas_operation_none,
                      ta ? rocblas_operation_transpose : rocblas_operation_none, n, m, k, &alpha, b.as_ptr(), ldb, a.as_ptr(), lda,
                      &beta, out.as_ptr(), n) != rocblas_status_success) {
        std::printf("rocblas_sgemm failed\n");
        std::exit(1);
    }
    return out;
}

struct Step {
    M x, t, neg_n, one;
    Parameters<float> p;       // name -> (param, grad)
    std::string wk[3], bk[3];
    Adam<float> *opt = nullptr;
    M loss;

    void init(const std::vector<float> &buf)
    {
        size_t o = 0;
        auto take = [&](Dim shape) {
            const size_t n = (size_t)num_elm(shape);
            M m = M::from_vec(std::vector<float>(buf.begin() + o, buf.begin() + o + n), shape);
            o += n;
            return m;
        };
        x = take({kBatch, 784});
        t = take({kBatch, 10});
        for (int i = 0; i < 3; i++) {
            wk[i] = "linear" + std::to_string(i + 1) + ".weight";
            bk[i] = "linear" + std::to_string(i + 1) + ".bias";
            p[wk[i]] = ParamGrad<float>(take({kLayers[i][1], kLayers[i][0]}));
            p[bk[i]] = ParamGrad<float>(take({kLayers[i][1]}));
        }
        neg_n = M::from_vec({-(float)kBatch}, {});
        one = M::from_vec({1.f}, {});
        opt = new Adam<float>(1e-3f, 0.9f, 0.999f, 1e-8f, p);
    }

    // `gb_in`: the bias gradient of the last layer when the caller's fused call has already produced it
    void backward_linears(M g, const M acts_in[3], const M Wt[3], const M pre[3], bool fused, M gb_in = M())
    {
        M gb_next = gb_in;
        for (int i = 2; i >= 0; i--) {
            M gb;
            if (fused) {
                gb = gb_next;                                           // came with the gradient, same launch
            } else {
                gb = M::zeros({kLayers[i][1]});
                g.sum_to(gb);                                           // bias gradient
            }
            M inT = acts_in[i].transpose().to_default_stride();
            M gWt = gemm(inT, g);                                       // dW^T = X^T dY
            p[wk[i]] = ParamGrad<float>(p[wk[i]].data, gWt.transpose().to_default_stride());
            p[bk[i]] = ParamGrad<float>(p[bk[i]].data, gb);
            if (i > 0) {
                M WtT = Wt[i].transpose().to_default_stride();
                M gh = gemm(g, WtT);                                    // dX = dY W
                if (fused) {
                    M gn = gh.alloc_like();
                    gb_next = M::alloc({kLayers[i - 1][1]});
                    gn.relu_backward_bias_grad(gb_next, gh, pre[i - 1], 0.f);
                    g = gn;
                } else {
                    M mask = pre[i - 1].alloc_like();
                    mask.relu_backward_mask(pre[i - 1], 0.f);
                    g = gh * mask;
                }
            }
        }
        opt->update(p);
    }

    // forward and backward with no materialised transpose: 20 launches
    void run_lean()
    {
        M pre[3], act_in[3];
        M h = x, logits;
        for (int i = 0; i < 3; i++) {
            act_in[i] = h;
            const int in = kLayers[i][0], out = kLayers[i][1];
            M z = gemm_rm(false, true, kBatch, out, in, h, in, p[wk[i]].data, in);      // h W^T, W stored [out, in]
            if (i == 2) {
                logits = z + p[bk[i]].data;
            } else {
                pre[i] = z.alloc_like();
                M a = z.alloc_like();
                a.bias_add_relu(z, p[bk[i]].data, 0.f, &pre[i]);
                h = a;
            }
        }
        auto lp = cross_entropy(logits, t);
        loss = lp.first;
        M gb = M::alloc({kLayers[2][1]});
        M g = cross_entropy_backward_bias_grad(lp.second, t, gb, &one);
        for (int i = 2; i >= 0; i--) {
            const int in = kLayers[i][0], out = kLayers[i][1];
            M gW = gemm_rm(true, false, out, in, kBatch, g, out, act_in[i], in);        // dY^T X, already [out, in]
            M w = p[wk[i]].data;
            p[wk[i]] = ParamGrad<float>(w, gW);
            p[bk[i]] = ParamGrad<float>(p[bk[i]].data, gb);
            if (i > 0) {
                M gh = gemm_rm(false, false, kBatch, in, out, g, out, w, in);           // dY W
                M gn = gh.alloc_like();
                gb = M::alloc({in});
                gn.relu_backward_bias_grad(gb, gh, pre[i - 1], 0.f);
                g = gn;
            }
        }
        opt->update(p);
    }

    void run(int variant)
    {
        if (variant == 2) return run_lean();
        const bool fused = variant == 1;
        M Wt[3], pre[3], act_in[3];
        M h = x;
        M logits;
        for (int i = 0; i < 3; i++) {
            act_in[i] = h;
            Wt[i] = p[wk[i]].data.transpose().to_default_stride();      // transpose(W): a materialised copy
            M z = gemm(h, Wt[i]);
            if (i == 2) {
                logits = z + p[bk[i]].data;
            } else if (fused) {
                pre[i] = z.alloc_like();
                M a = z.alloc_like();
                a.bias_add_relu(z, p[bk[i]].data, 0.f, &pre[i]);
                h = a;
            } else {
                pre[i] = z + p[bk[i]].data;
                M a = pre[i].alloc_like();
                a.relu(pre[i], 0.f);
                h = a;
            }
        }
        M g, gb_last;
        if (fused) {
            auto lp = cross_entropy(logits, t);
            loss = lp.first;
            gb_last = M::alloc({kLayers[2][1]});
            g = cross_entropy_backward_bias_grad(lp.second, t, gb_last, &one);
        } else {
            M diff = logits - logits.max_axis(1, true);                 // softmax_assign
            M e = diff.exp();
            e /= e.sum(1, true);
            M s = e.alloc_like();
            s.copy_from(e);
            M yl = t * s.log();                                         // cross_entropy
            M total = M::zeros({});
            yl.sum_to(total);
            loss = total / neg_n;
            M g_total = one / neg_n;                                    // backward of div, sum_to, mul, log, softmax
            M g_yl = M::zeros({kBatch, 10});
            g_yl += g_total;
            M g_s = (t * g_yl) / s;
            M gx = s * g_s;
            g = gx - s * gx.sum(1, true);
        }
        backward_linears(g, act_in, Wt, pre, fused, gb_last);
    }
};

static std::vector<float> synthetic()
{
    size_t n = (size_t)kBatch * 784 + kBatch * 10;
    for (auto &l : kLayers) n += (size_t)l[0] * l[1] + l[1];
    std::vector<float> buf(n, 0.f);
    uint64_t s = 88172645463325252ull;
    auto u01 = [&]() {
        s ^= s << 13; s ^= s >> 7; s ^= s << 17;
        return (float)((s >> 11) * (1.0 / 9007199254740992.0));
    };
    size_t o = 0;
    for (int i = 0; i < kBatch * 784; i++) buf[o++] = u01();
    for (int r = 0; r < kBatch; r++) {
        buf[o + r * 10 + (int)(u01() * 10) % 10] = 1.f;
    }
    o += kBatch * 10;
    for (auto &l : kLayers) {
        const float sc = 1.f / std::sqrt((float)l[0]);
        for (int i = 0; i < l[0] * l[1]; i++) buf[o++] = (u01() + u01() + u01() + u01() - 2.f) * 1.7320508f * sc;  // ~N(0,1)/sqrt(fan_in)
        o += l[1];                                                                                                  // bias 0
    }
    return buf;
}

int main(int argc, char **argv)
{
    std::string inputs;
    int steps = 50, warmup = 5, dump = 0;
    for (int i = 1; i < argc; i++) {
        if (!std::strcmp(argv[i], "--inputs") && i + 1 < argc) inputs = argv[++i];
        else if (!std::strcmp(argv[i], "--steps") && i + 1 < argc) steps = std::atoi(argv[++i]);
        else if (!std::strcmp(argv[i], "--warmup") && i + 1 < argc) warmup = std::atoi(argv[++i]);
        else if (!std::strcmp(argv[i], "--dump-loss") && i + 1 < argc) dump = std::atoi(argv[++i]);
    }
    std::vector<float> buf = synthetic();
    if (!inputs.empty()) {
        FILE *f = std::fopen(inputs.c_str(), "rb");
        if (!f || std::fread(buf.data(), sizeof(float), buf.size(), f) != buf.size()) {
            std::printf("cannot read %s\n", inputs.c_str());
            return 1;
        }
        std::fclose(f);
    }
    try {
        init(0);
        zenu_stream_t stream;
        check(zenu_hip_stream_create(&stream), "stream_create");
        current_stream() = stream;
        if (rocblas_create_handle(&g_blas) != rocblas_status_success ||
            rocblas_set_stream(g_blas, reinterpret_cast<hipStream_t>(stream)) != rocblas_status_success) {
            std::printf("rocblas init failed\n");
            return 1;
        }
        {   // what one launch costs when the kernel does next to nothing: one-element adds issued back to
            // back through the C ABI (the rate at which the HIP runtime and the dispatcher hand out kernels)
            zenu_hip::Matrix<float> a = zenu_hip::Matrix<float>::zeros({1}), b = zenu_hip::Matrix<float>::zeros({1}),
                                    c = zenu_hip::Matrix<float>::zeros({1});
            zenu_tensor_t ta = a.desc(), tb = b.desc(), tc = c.desc();
            const int n = 20000;
            for (int i = 0; i < 2000; i++) zenu_hip_binary(ZENU_ADD, ZENU_F32, &tc, &ta, &tb, stream);
            synchronize();
            const auto t0 = std::chrono::steady_clock::now();
            for (int i = 0; i < n; i++) zenu_hip_binary(ZENU_ADD, ZENU_F32, &tc, &ta, &tb, stream);
            synchronize();
            std::printf("floor launch_us %.3f\n", std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() / n);
        }
        for (int fused = 0; fused < 3; fused++) {
            const char *name = fused == 2 ? "lean" : fused ? "fused" : "ops";
            Step st;
            st.init(buf);
            for (int i = 0; i < dump; i++) {            // the first steps' losses, for the parity test
                st.run(fused);
                std::printf("%s loss %d %.9g\n", name, i + 1, (double)st.loss.to_vec()[0]);
            }
            for (int i = 0; i < warmup; i++) st.run(fused);
            synchronize();
            const auto t0 = std::chrono::steady_clock::now();
            for (int i = 0; i < steps; i++) st.run(fused);
            // time the host needed to issue the steps (it runs ahead of the GPU until the queue is full)
            const double issue_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / steps;
            synchronize();
            const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / steps;
            std::printf("%s ms_per_step %.4f\n", name, ms);
            std::printf("%s host_issue_ms_per_step %.4f\n", name, issue_ms);
            std::printf("%s final_loss %.9g\n", name, (double)st.loss.to_vec()[0]);
            std::fflush(stdout);
        }
    } catch (const std::exception &e) {
        std::printf("FAILED %s\n", e.what());
        return 1;
    }
    return 0;
}
