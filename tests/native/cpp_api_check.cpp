// The reference's known-answer tests, written against the C++ host API (include/zenu_hip.hpp) the
// way the reference writes them against Matrix<_, DimDyn, D>.  Each case names the Rust test it
// restates; where a line is cited the inputs and expected values are that test's literals, a few
// cases (sub_mul_div, sum_4d, copy_cases, the tie rows) build the expectation from the same
// definition with host arithmetic.  Prints "ok <case>" per case and exits non-zero on the first failure.  Needs a GPU (run by tests/test_cpp_api.py).
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <string>

#include "zenu_hip.hpp"

using namespace zenu_hip;
typedef Matrix<float> M;
typedef Matrix<double> Md;

static void fail(const char *what, int line)
{
    std::printf("FAILED %s (line %d)\n", what, line);
    std::fflush(stdout);
    std::exit(1);
}
#define REQUIRE(c) do { if (!(c)) fail(#c, __LINE__); } while (0)

template <typename T> static bool eq(const Matrix<T> &m, const std::vector<T> &exp)
{
    return m.to_vec() == exp;
}
template <typename T> static bool close(const Matrix<T> &m, const std::vector<double> &exp, double eps)
{
    std::vector<T> v = m.to_vec();
    if (v.size() != exp.size()) return false;
    for (size_t i = 0; i < v.size(); i++)
        if (!(std::fabs((double)v[i] - exp[i]) <= eps)) return false;
    return true;
}
static std::vector<float> iota(int n, float first = 1.f)
{
    std::vector<float> v(n);
    for (int i = 0; i < n; i++) v[i] = first + i;
    return v;
}
template <typename F> static bool throws_status(int status, F f)
{
    try {
        f();
    } catch (const Error &e) {
        return e.status == status;
    }
    return false;
}

// ---- zenu-matrix/src/operation/basic_operations.rs ------------------------------------------------------------

static void scalar_add_2d()   // :667
{
    M a = M::from_vec({1, 2, 3, 4, 5, 6}, {2, 3});
    M ans = M::zeros({2, 3});
    ans.add_scalar(a, 1.f);
    REQUIRE(eq(ans, {2, 3, 4, 5, 6, 7}));
}

static void sliced_3d()       // :689  slice_dynamic!(1.., .., ..;2)
{
    M a = M::from_vec(iota(16), {2, 2, 4});
    M ans = M::zeros({1, 2, 2});
    ans.add_scalar(a.slice({Slice(1, -1), Slice(), Slice(0, -1, 2)}), 1.f);
    REQUIRE(eq(ans, {10, 12, 14, 16}));
}

static void sliced_3d_assign()   // :749  slice_dynamic!(2, 1..3, ..;2)
{
    std::vector<float> v;
    for (int i = 0; i < 3; i++)
        for (int j = 0; j < 4; j++)
            for (int k = 0; k < 5; k++) v.push_back((float)(i * 100 + j * 10 + k));
    M a = M::from_vec(v, {3, 4, 5}).index_axis(0, 2).slice({Slice(1, 3), Slice(0, -1, 2)});
    M ans = M::zeros({2, 3});
    ans.add_scalar(a, 1.f);
    REQUIRE(eq(ans, {211, 213, 215, 221, 223, 225}));
}

static void matrix_add_sliced()   // :823
{
    M a = M::from_vec(iota(16), {4, 4}).slice({Slice(1, -1, 2), Slice(0, -1, 2)});
    M b = M::from_vec(iota(16), {4, 4}).slice({Slice(0, -1, 2), Slice(1, -1, 2)});
    M ans = M::zeros({2, 2});
    ans.add_array(a, b);
    REQUIRE(eq(ans, {7, 11, 23, 27}));
}

static void transposed()      // :856-889
{
    M a = M::from_vec(iota(16), {4, 4}).transpose();
    M b = M::from_vec(iota(16), {4, 4});
    M ans = M::zeros({4, 4});
    ans.add_array(a, b);
    REQUIRE(eq(ans, {2, 7, 12, 17, 7, 12, 17, 22, 12, 17, 22, 27, 17, 22, 27, 32}));
}

static void broadcast_add()   // :900, :925, :950
{
    M a = M::from_vec({1, 2, 3, 4}, {2, 2});
    M b = M::from_vec({1, 2}, {2});
    M ans = M::zeros({2, 2});
    ans.add_array(a, b);
    REQUIRE(eq(ans, {2, 4, 4, 6}));
    M s = M::from_vec({3}, {});
    ans.add_array(a, s);
    REQUIRE(eq(ans, {4, 5, 6, 7}));
    REQUIRE(eq(a + s, {4, 5, 6, 7}));      // impl_ops.rs: a 0-d operand is a device-side scalar
}

static void broadcast_add_1x4x1x1_3x4x5x5()   // :1005
{
    M a = M::from_vec({1, 2, 3, 4}, {1, 4, 1, 1});
    M b = M::zeros({3, 4, 5, 5});
    M ans = M::zeros({3, 4, 5, 5});
    ans.add_array(a, b);
    std::vector<float> exp(300);
    for (int i = 0; i < 300; i++) exp[i] = (float)((i / 25) % 4 + 1);
    REQUIRE(eq(ans, exp));
}

static void sub_mul_div()     // :1035-1335
{
    M a = M::from_vec(iota(8), {2, 2, 2});
    M b = M::from_vec({2, 2, 2, 2, 4, 4, 4, 4}, {2, 2, 2});
    REQUIRE(eq(a - b, {-1, 0, 1, 2, 1, 2, 3, 4}));
    REQUIRE(eq(a * b, {2, 4, 6, 8, 20, 24, 28, 32}));
    REQUIRE(eq(a / b, {0.5f, 1, 1.5f, 2, 1.25f, 1.5f, 1.75f, 2}));
    REQUIRE(eq(a * 2.f, {2, 4, 6, 8, 10, 12, 14, 16}));
    M c = a.new_matrix();
    c.div_scalar_assign(2.f);
    REQUIRE(eq(c, {0.5f, 1, 1.5f, 2, 2.5f, 3, 3.5f, 4}));
    c -= a;
    REQUIRE(eq(c, {-0.5f, -1, -1.5f, -2, -2.5f, -3, -3.5f, -4}));
}

static void shape_errors()    // with_clousers.rs:87-107,155-178
{
    M a = M::zeros({2, 3}), b = M::zeros({3, 2}), out = M::zeros({2, 3});
    REQUIRE(throws_status(ZENU_ERR_SHAPE, [&] { out.add_array(a, b); }));
    REQUIRE(throws_status(ZENU_ERR_SHAPE, [&] { a.copy_from(b); }));
    REQUIRE(throws_status(ZENU_ERR_AXIS, [&] { a.sum(2); }));
}

// ---- unary, relu, sigmoid ----------------------------------------------------------------------------------------

static void unary_tables()    // zenu-cuda/src/kernel/mod.rs:1015-1241, 1e-6
{
    M a = M::from_vec({0, 1, 2, 3}, {4});
    REQUIRE(close(a.exp(), {1.0, 2.718281828, 7.389056099, 20.08553692}, 2e-6 * 20));
    M b = M::from_vec({1, 2, 3, 4}, {4});
    REQUIRE(close(b.log(), {0.0, 0.693147181, 1.098612289, 1.386294361}, 1e-6));
    REQUIRE(close(a.tanh(), {0.0, 0.761594156, 0.96402758, 0.995054754}, 1e-6));
    REQUIRE(close(a.tanh_ulp2(), {0.0, 0.761594156, 0.96402758, 0.995054754}, 1e-6));   // the 2-ulp variant, same table
    REQUIRE(close(b.sqrt(), {1.0, 1.414213562, 1.732050808, 2.0}, 1e-6));
    M c = M::from_vec({-1, 2, -3, 4}, {4});
    REQUIRE(eq(c.abs(), {1, 2, 3, 4}));
    c.abs_assign();
    REQUIRE(eq(c, {1, 2, 3, 4}));
}

static void relu_cases()      // relu.rs:255-296, kernel/activation.rs:88-147
{
    M x = M::from_vec({1, -1, 0, 2, -2}, {5});
    M y = M::zeros({5});
    y.relu(x, 0.2f);
    REQUIRE(close(y, {1, -0.2, 0, 2, -0.4}, 1e-7));
    y.relu_backward_mask(x, 0.1f);
    REQUIRE(close(y, {1, -0.1, -0.1, 1, -0.1}, 1e-7));
}

static void sigmoid_cases()   // zenu-autograd/src/activation/sigmoid.rs:26-66
{
    M x = M::from_vec({0.f, 0.5f, 0.1f}, {3});
    REQUIRE(close(x.sigmoid(), {0.5, 0.62245935, 0.52497919}, 1e-6));
}

// ---- reductions ----------------------------------------------------------------------------------------------------

static void sum_4d()          // sum.rs:109-245
{
    M a = M::from_vec(iota(120, 0.f), {2, 3, 4, 5});
    M s0 = a.sum(0);
    std::vector<float> exp(60);
    for (int i = 0; i < 60; i++) exp[i] = (float)(i + (i + 60));
    REQUIRE(eq(s0, exp));
    M s3 = a.sum(3, true);
    REQUIRE((s3.shape() == Dim{2, 3, 4, 1}));
    std::vector<float> exp3(24);
    for (int i = 0; i < 24; i++) exp3[i] = (float)(5 * (5 * i) + 10);
    REQUIRE(eq(s3, exp3));
    M tot = M::zeros({});
    a.sum_to(tot);
    REQUIRE(eq(tot, {7140.f}));
    REQUIRE(eq(a.sum_all(), {7140.f}));
    // the entry point that allocates nothing gives the same sums into an existing matrix
    M s0b = M::zeros({3, 4, 5});
    a.sum_noalloc(0, s0b);
    REQUIRE(eq(s0b, exp));
    REQUIRE(zenu_hip::last_status() == ZENU_OK);
}

static void max_cases()       // max.rs:157-245
{
    REQUIRE((M::from_vec({0, 1, 2, 3}, {4}).max_idx() == Dim{3}));
    M b = M::from_vec({0, 1, 2, 3}, {2, 2});
    REQUIRE((b.max_idx() == Dim{1, 1}));
    M c = M::from_vec(iota(512, 0.f), {8, 8, 8});
    M sl = c.slice({Slice(0, -1, 3), Slice(0, -1, 4), Slice(0, -1, 2)});   // ..;3, ..;4, ..;2
    REQUIRE((sl.max_idx() == Dim{2, 1, 3}));
    REQUIRE(sl.max_item() == (float)(6 * 64 + 4 * 8 + 6));
    // max_axis_reval :204-245
    Md d = Md::from_vec({0.04881350392732475, 0.21518936637241948, 0.10276337607164387, 0.044883182996896864,
                         -0.07634520066109529, 0.14589411306665612, -0.06241278873730749, 0.39177300078207977,
                         0.4636627605010293, -0.1165584811742223, 0.2917250380826646, 0.02889491975290448,
                         0.06804456109393231, 0.42559663829266103, -0.42896394180211306, -0.4128707002984593,
                         -0.4797816025596743, 0.332619845547938, 0.2781567509498505, 0.37001214824681916,
                         0.478618342232764, 0.2991585642167236, -0.038520637747068154, 0.28052917628645546}, {2, 3, 4});
    REQUIRE((d.max_axis_idx_ravel(0) == std::vector<int64_t>{1, 1, 0, 0, 0, 1, 1, 0, 1, 1, 0, 1}));
    REQUIRE((d.max_axis_idx_ravel(1) == std::vector<int64_t>{2, 0, 2, 1, 2, 0, 1, 1}));
    REQUIRE((d.max_axis_idx_ravel(2) == std::vector<int64_t>{1, 3, 0, 1, 3, 0}));
    // ties: the first index wins (max.rs:27, strict '>'); no reference test has ties
    M t = M::from_vec({1, 7, 7, 3, 7, 7, 7, 7}, {2, 4});
    REQUIRE((t.max_axis_idx_ravel(1) == std::vector<int64_t>{1, 0}));
    REQUIRE(eq(t.max_axis(1), {7, 7}));
}

static void asum_cases()      // asum.rs:78-120
{
    REQUIRE(M::from_vec({1, 2, 3}, {3}).asum() == 6.f);
    M a = M::from_vec({1, 2, 3, 4}, {2, 2});
    REQUIRE(a.asum() == 10.f);
    REQUIRE(a.slice({Slice(0, 2), Slice(0, 1)}).asum() == 4.f);
}

static void copy_cases()      // copy_from.rs:285-398, to_default_stride.rs:28-89
{
    M a = M::from_vec(iota(12, 0.f), {3, 4});
    M t = a.transpose().to_default_stride();
    REQUIRE((t.shape() == Dim{4, 3}));
    REQUIRE(eq(t, {0, 4, 8, 1, 5, 9, 2, 6, 10, 3, 7, 11}));
    M big = M::zeros({3, 8});
    big.slice({Slice(), Slice(0, -1, 2)}).copy_from(a);
    REQUIRE(big.index_item({2, 6}) == 11.f);
    REQUIRE(big.index_item({2, 5}) == 0.f);
    REQUIRE(eq(a.index_axis(0, 1), {4, 5, 6, 7}));
    REQUIRE(eq(a.reshape({2, 6}).index_axis(1, 5), {5, 11}));
    REQUIRE(eq(a.add_axis(0).index_axis(0, 0).index_axis(1, 3), {3, 7, 11}));
    REQUIRE(eq(a.transpose_by_index({1, 0}), t.to_vec()));
}

static void broadcast_cases() // broadcast.rs:53-165
{
    M src = M::from_vec({1, 2}, {1, 2});
    M res = M::zeros({2, 3, 1, 2});
    res.broadcast(src);
    REQUIRE(eq(res, {1, 2, 1, 2, 1, 2, 1, 2, 1, 2, 1, 2}));
    M s0 = M::from_vec({1}, {});
    M r1 = M::zeros({3});
    r1.broadcast(s0);
    REQUIRE(eq(r1, {1, 1, 1}));
}

static void stack_split_cases() // stack.rs:71-108, split.rs:70-117
{
    std::vector<M> v1 = {M::from_vec({1, 2, 3}, {3}), M::from_vec({4, 5, 6}, {3}), M::from_vec({7, 8, 9}, {3})};
    REQUIRE(eq(stack(v1, 0), {1, 2, 3, 4, 5, 6, 7, 8, 9}));
    std::vector<M> v2 = {M::from_vec({1, 2, 3, 4}, {2, 2}), M::from_vec({5, 6, 7, 8}, {2, 2}), M::from_vec({9, 10, 11, 12}, {2, 2})};
    M s = stack(v2, 1);
    REQUIRE(s.shape() == Dim({2, 6}));
    REQUIRE(eq(s, {1, 2, 5, 6, 9, 10, 3, 4, 7, 8, 11, 12}));
    std::vector<M> p0 = split(M::from_vec({1, 2, 3, 4, 5, 6}, {3, 2}), 0, 3);
    REQUIRE(p0.size() == 3 && p0[0].shape() == Dim({1, 2}) && eq(p0[0], {1, 2}) && eq(p0[1], {3, 4}) && eq(p0[2], {5, 6}));
    std::vector<M> p1 = split(M::from_vec({1, 2, 3, 4, 5, 6}, {2, 3}), 1, 3);
    REQUIRE(p1[0].shape() == Dim({2, 1}) && eq(p1[0], {1, 4}) && eq(p1[1], {2, 5}) && eq(p1[2], {3, 6}));
    REQUIRE(throws_status(ZENU_ERR_SHAPE, [&] { split(M::from_vec({1, 2, 3}, {3}), 0, 2); }));
}

static void mean_variance_cases() // var.rs test mod, mean.rs:9-20
{
    REQUIRE(close(M::from_vec({1, 2, 3, 4}, {4}).variance_all(), {1.25}, 1e-6));
    REQUIRE(close(M::from_vec({1, 2}, {2}).variance_all(), {0.25}, 1e-6));
    M x = M::from_vec({1, 2, 3, 4}, {2, 2});
    REQUIRE(close(x.variance_all(), {1.25}, 1e-6));
    REQUIRE(close(x.variance(0), {1., 1.}, 1e-6));
    REQUIRE(close(x.variance(1), {0.25, 0.25}, 1e-6));
    REQUIRE(close(x.mean(1, true), {1.5, 3.5}, 1e-6));
    REQUIRE(close(M::from_vec({-1, 2, -3, 4}, {4}).mean_all(), {2.5}, 1e-6));   // the mean of |x|
}

static void conv_bias_cases() // zenu-matrix/src/nn/conv/mod.rs:84-107, cpu/bias.rs:10-25
{
    const int n = 2, c = 3, h = 2, w = 4;
    M x = M::from_vec(iota(n * c * h * w), {n, c, h, w});
    M b = M::from_vec({10, 20, 30}, {1, c, 1, 1});
    M y = M::zeros({n, c, h, w});
    conv2d_bias_add(x, b, y);
    std::vector<float> exp = iota(n * c * h * w);
    std::vector<float> gexp(c, 0.f);
    for (int i = 0; i < n * c * h * w; i++) {
        const int ch = (i / (h * w)) % c;
        gexp[ch] += exp[i];            // small integers: exact in any order
        exp[i] += 10.f * (ch + 1);
    }
    REQUIRE(eq(y, exp));
    M g = M::zeros({1, c, 1, 1});
    conv2d_bias_bkwd(x, g);
    REQUIRE(eq(g, gexp));
    REQUIRE(throws_status(ZENU_ERR_SHAPE, [&] { conv2d_bias_bkwd(x, M::zeros({c})); }));
}

// ---- softmax, cross-entropy, clip ----------------------------------------------------------------------------------

static void softmax_cases()   // softmax.rs:37-91; loss/softmax.rs:70-103
{
    M a = M::from_vec({1, 2, 3, 4, 5, 6}, {2, 3});
    M b = M::zeros({2, 3});
    b.softmax_assign(a, 1);
    REQUIRE(close(b, {0.09003057, 0.24472847, 0.66524096, 0.09003057, 0.24472847, 0.66524096}, 1e-6));
    b.softmax_assign(a, 0);
    REQUIRE(close(b, {0.04742587, 0.04742587, 0.04742587, 0.95257413, 0.95257413, 0.95257413}, 1e-6));
    Md x = Md::from_vec({1, 2, 3, 4, 5, 6, 7, 8}, {2, 4});
    Md y = Md::zeros({2, 4});
    y.softmax_assign(x, 1);
    Md gy = Md::from_vec({1, 2, 3, 4, 1, 2, 3, 4}, {2, 4});
    REQUIRE(close(softmax_backward(y, gy, 1),
                  {-0.07991097, -0.13007621, -0.11670097, 0.32668814, -0.07991097, -0.13007621, -0.11670097, 0.32668814}, 1e-6));
}

static void cross_entropy_cases()   // loss/cross_entropy.rs:38-84
{
    M pred = M::from_vec({0.1f, 0.9f, 0.1f, 0.1f, 0.01f, 0.9f, 0.2f, 0.05f}, {2, 4});
    M ans = M::from_vec({0, 1, 0, 0, 1, 0, 0, 0}, {2, 4});
    auto lp = cross_entropy(pred, ans);
    REQUIRE(close(lp.first, {1.2957}, 2e-5));
    REQUIRE(close(cross_entropy_backward(lp.second, ans), {0.0957, -0.2871, 0.0957, 0.0957, -0.4121, 0.2142, 0.1064, 0.0915}, 3e-4));
}

static void clip_cases()      // clip.rs:321-372; kernel/mod.rs:1300-1368
{
    M a = M::from_vec({1, 2, 3, 4}, {2, 2});
    REQUIRE(eq(a.clip(2.f, 3.f), {2, 2, 3, 3}));
    a.clip_assign(2.f, 3.f);
    REQUIRE(eq(a, {2, 2, 3, 3}));
    Md b = Md::from_vec({0, 1, 2, 3, 4, 5}, {6});
    REQUIRE(eq(b.clip_backward_mask(1.0, 2.0), {0, 1, 1, 0, 0, 0}));
}

// ---- optimizers: zenu-optimizer/tests/net_test.rs ---------------------------------------------------------------------
// SimpleNet: y = Linear2(Linear1(x)), y = x W^T + b (zenu-layer/src/layers/linear.rs:19-32);
// loss = sum((t - y)^2) / t.shape[0] (zenu-autograd/src/loss/mse.rs:6-14).  Weights, input and target are
// the literals of net_test.rs:93-105; the forward/backward of the tiny net is written out with library
// ops (the two matrix products as broadcast multiply + sum), the update is the optimizer under test.

static const char *kW1 = "linear1.linear.weight", *kB1 = "linear1.linear.bias";
static const char *kW2 = "linear2.linear.weight", *kB2 = "linear2.linear.bias";

struct Net {
    Parameters<float> p;
    M x, t;
    Net()
    {
        p[kW1] = ParamGrad<float>(M::from_vec({0.1f, 0.2f, 0.3f, 0.4f, 0.5f, 0.6f, 0.07f, 0.08f}, {4, 2}));
        p[kB1] = ParamGrad<float>(M::from_vec({0.1f, 0.2f, 0.3f, 0.4f}, {4}));
        p[kW2] = ParamGrad<float>(M::from_vec({0.1f, 0.2f, 0.3f, 0.4f, 0.5f, 0.6f, 0.07f, 0.08f, 0.09f, 0.10f, 0.11f, 0.12f,
                                               0.13f, 0.14f, 0.15f, 0.16f}, {4, 4}));
        p[kB2] = ParamGrad<float>(M::from_vec({0.1f, 0.2f, 0.3f, 0.4f}, {4}));
        x = M::from_vec({0.1f, 0.2f}, {1, 2});
        t = M::from_vec({0.1f, 0.2f, 0.3f, 0.4f}, {1, 4});
    }
    // y[1,out] = sum_k x[1,k] * W[out,k] + b
    static M linear(const M &x, const M &W, const M &b) { return (W * x).sum(1).add_axis(0) + b; }
    void backward()
    {
        const M W1 = p[kW1].data, b1 = p[kB1].data, W2 = p[kW2].data, b2 = p[kB2].data;
        M h = linear(x, W1, b1);
        M y = linear(h, W2, b2);
        M gy = (y - t) * (2.f / 4.f);
        M gyT = gy.transpose().to_default_stride();         // [4,1]
        M gW2 = M::zeros({4, 4});
        gW2.broadcast(h);                                   // every row = h
        gW2 *= gyT;                                         // gy^T h
        M gh = (W2 * gyT).sum(0).add_axis(0);               // sum_o gy[o] * W2[o,k] -> [1,4]
        M ghT = gh.transpose().to_default_stride();
        M gW1 = M::zeros({4, 2});
        gW1.broadcast(x);
        gW1 *= ghT;
        p[kW2] = ParamGrad<float>(W2, gW2);
        p[kB2] = ParamGrad<float>(b2, gy.index_axis(0, 0).new_matrix());
        p[kW1] = ParamGrad<float>(W1, gW1);
        p[kB1] = ParamGrad<float>(b1, gh.index_axis(0, 0).new_matrix());
    }
    bool matches(const std::vector<double> &w1, const std::vector<double> &b1, const std::vector<double> &w2,
                 const std::vector<double> &b2, double eps)
    {
        return close(p[kW1].data, w1, eps) && close(p[kB1].data, b1, eps) && close(p[kW2].data, w2, eps) &&
               close(p[kB2].data, b2, eps);
    }
};

static void sgd_net_test()    // net_test.rs:107-141: lr 0.9, one step, 1e-4
{
    Net net;
    net.backward();
    SGD<float>(0.9f).update(net.p);
    REQUIRE(net.matches({0.0891, 0.1782, 0.2857, 0.3715, 0.4917, 0.5833, 0.0596, 0.0592}, {-0.0089, 0.0574, 0.2166, 0.2961},
                        {0.0739, 0.1460, 0.2181, 0.3263, 0.4779, 0.5543, 0.0007, 0.0176, 0.0801, 0.0795, 0.0789, 0.0920,
                         0.1164, 0.1119, 0.1075, 0.1217}, {-0.0742, 0.0525, 0.2339, 0.3095}, 1e-4));
}

static void adam_net_test()   // net_test.rs:143-189: two optimizers, each takes its first step, 2e-4
{
    Net net;
    for (int i = 0; i < 2; i++) {
        net.backward();
        Adam<float>(0.01f, 0.9f, 0.999f, 1e-8f, net.p).update(net.p);
    }
    REQUIRE(net.matches({0.0801, 0.1801, 0.2801, 0.3801, 0.4801, 0.5801, 0.0501, 0.0601}, {0.0801, 0.1801, 0.2801, 0.3801},
                        {0.0801, 0.1801, 0.2801, 0.3801, 0.4801, 0.5801, 0.0501, 0.0601, 0.0702, 0.0801, 0.0901, 0.1001,
                         0.1101, 0.1201, 0.1301, 0.1401}, {0.0800, 0.1801, 0.2801, 0.3801}, 2e-4));
}

static void adam_w_net_test() // net_test.rs:191-232: one optimizer, two steps, weight decay 0.01 on the weights, 2e-4
{
    Net net;
    AdamW<float> opt(0.01f, 0.9f, 0.999f, 1e-8f, 0.01f, net.p, {kW1, kW2});
    for (int i = 0; i < 2; i++) {
        net.backward();
        opt.update(net.p);
    }
    REQUIRE(net.matches({0.0801, 0.1800, 0.2800, 0.3800, 0.4800, 0.5800, 0.0501, 0.0601}, {0.0801, 0.1800, 0.2800, 0.3800},
                        {0.0801, 0.1800, 0.2800, 0.3800, 0.4800, 0.5800, 0.0501, 0.0601, 0.0702, 0.0801, 0.0901, 0.1001,
                         0.1101, 0.1201, 0.1301, 0.1401}, {0.0800, 0.1800, 0.2801, 0.3800}, 2e-4));
}

static void adam_w_net_test_scheduled()   // the same two steps with the step-dependent scalars in device memory
{
    Net net;
    AdamW<float> opt(0.01f, 0.9f, 0.999f, 1e-8f, 0.01f, net.p, {kW1, kW2});
    opt.use_schedule(2);
    for (int i = 0; i < 2; i++) {
        net.backward();
        opt.update(net.p);
    }
    REQUIRE(net.matches({0.0801, 0.1800, 0.2800, 0.3800, 0.4800, 0.5800, 0.0501, 0.0601}, {0.0801, 0.1800, 0.2800, 0.3800},
                        {0.0801, 0.1800, 0.2800, 0.3800, 0.4800, 0.5800, 0.0501, 0.0601, 0.0702, 0.0801, 0.0901, 0.1001,
                         0.1101, 0.1201, 0.1301, 0.1401}, {0.0800, 0.1800, 0.2801, 0.3800}, 2e-4));
    int64_t next = 0, left = 0, refused = 0;
    opt.schedule_state(next, left, refused);
    REQUIRE(next == 3 && left == 0 && refused == 0);
    net.backward();
    opt.update(net.p);                        // past the end of the table: nothing changes, and it is counted
    opt.schedule_state(next, left, refused);
    REQUIRE(next == 3 && refused == 1);
    REQUIRE(net.matches({0.0801, 0.1800, 0.2800, 0.3800, 0.4800, 0.5800, 0.0501, 0.0601}, {0.0801, 0.1800, 0.2800, 0.3800},
                        {0.0801, 0.1800, 0.2800, 0.3800, 0.4800, 0.5800, 0.0501, 0.0601, 0.0702, 0.0801, 0.0901, 0.1001,
                         0.1101, 0.1201, 0.1301, 0.1401}, {0.0800, 0.1800, 0.2801, 0.3800}, 2e-4));
}

int main(int argc, char **argv)
{
    init(0);
    struct Case { const char *name; std::function<void()> fn; };
    const Case cases[] = {
        {"scalar_add_2d", scalar_add_2d}, {"sliced_3d", sliced_3d}, {"sliced_3d_assign", sliced_3d_assign},
        {"matrix_add_sliced", matrix_add_sliced},
        {"transposed", transposed}, {"broadcast_add", broadcast_add},
        {"broadcast_add_1x4x1x1_3x4x5x5", broadcast_add_1x4x1x1_3x4x5x5}, {"sub_mul_div", sub_mul_div},
        {"shape_errors", shape_errors}, {"unary_tables", unary_tables}, {"relu_cases", relu_cases},
        {"sigmoid_cases", sigmoid_cases}, {"sum_4d", sum_4d}, {"max_cases", max_cases}, {"asum_cases", asum_cases},
        {"copy_cases", copy_cases}, {"broadcast_cases", broadcast_cases}, {"conv_bias_cases", conv_bias_cases}, {"mean_variance_cases", mean_variance_cases}, {"stack_split_cases", stack_split_cases},
        {"softmax_cases", softmax_cases},
        {"cross_entropy_cases", cross_entropy_cases}, {"clip_cases", clip_cases}, {"sgd_net_test", sgd_net_test},
        {"adam_net_test", adam_net_test}, {"adam_w_net_test", adam_w_net_test},
        {"adam_w_net_test_scheduled", adam_w_net_test_scheduled},
    };
    for (const Case &c : cases) {
        if (argc > 1 && std::string(argv[1]) != c.name) continue;
        std::printf("[case] %s\n", c.name);
        std::fflush(stdout);
        try {
            c.fn();
        } catch (const std::exception &e) {
            std::printf("FAILED %s: %s\n", c.name, e.what());
            return 1;
        }
        std::printf("ok %s\n", c.name);
        std::fflush(stdout);
    }
    synchronize();
    return 0;
}
