#pragma once
// Known-answer cases for the public operator API, written once and run on the
// host cores and on the GPU.  Each case mirrors a test of xyz-autodiff-cuda (cited
// at the case) and writes the values that test inspects into out[]; the
// expectations live in tests/test_api_known_answers.py.
#include <xyz_autodiff/xyz_autodiff.cuh>
#include <xyz_autodiff/operations/unary/broadcast_logic.cuh>
#include <operations/covariance_generation.cuh>
#include <operations/mahalanobis_distance.cuh>

namespace xad_test {

using namespace xyz_autodiff;

constexpr int kCaseCapacity = 64;

// A user-written logic, as users of the library write them: y = x + c
// (the shape of tests/operation/unary/test_add_constant_operations_gradient.cu:98-118).
template <std::size_t Dim>
struct UserShiftLogic {
    static constexpr std::size_t outputDim = Dim;
    double c;
    template <typename Output, typename Input>
    XAD_HD void forward(Output& out, const Input& in) const {
        for (std::size_t i = 0; i < Dim; ++i) out[i] = in[i] + typename Input::value_type(c);
    }
    template <typename Output, typename Input>
    XAD_HD void backward(const Output& out, Input& in) const {
        for (std::size_t i = 0; i < Dim; ++i) in.add_grad(i, out.grad(i));
    }
};

// A user-written node that follows the three-call protocol of the reference
// (forward / increment_ref_count / decrement_ref_count_and_check) and knows
// nothing about this library's own traversal: y = 2 x over one operand.
template <typename Input>
class UserDoubleNode {
public:
    using value_type = typename Input::value_type;
    static constexpr std::size_t size = Input::size;
    XAD_HD explicit UserDoubleNode(Input& in) : in_(in) {}
    XAD_HD void forward() {
        if constexpr (OperationNode<Input>) {
            in_.forward();
            in_.increment_ref_count();
        }
        for (std::size_t i = 0; i < size; ++i) out_[i] = value_type(2) * in_[i];
    }
    XAD_HD void backward() {
        for (std::size_t i = 0; i < size; ++i) in_.add_grad(i, value_type(2) * out_.grad(i));
        if constexpr (OperationNode<Input>) {
            if (in_.decrement_ref_count_and_check()) in_.backward();
        }
    }
    XAD_HD void backward_numerical(value_type) { backward(); }
    XAD_HD void increment_ref_count() { ++count_; }
    XAD_HD bool decrement_ref_count_and_check() { return --count_ == 0; }
    XAD_HD value_type& operator[](std::size_t i) { return out_[i]; }
    XAD_HD const value_type& operator[](std::size_t i) const { return out_[i]; }
    XAD_HD const value_type& grad(std::size_t i) const { return out_.grad(i); }
    XAD_HD void add_grad(std::size_t i, value_type g) { out_.add_grad(i, g); }
    XAD_HD void zero_grad() { out_.zero_grad(); }

private:
    Input& in_;
    Variable<size, value_type> out_;
    unsigned char count_ = 0;
};

// A user-written three-operand logic: y = a * b + c, element-wise (the contract of
// TernaryLogicConcept, include/xyz_autodiff/concept/core_logic.cuh:44-54 of the reference).
template <std::size_t Dim>
struct UserMulAddLogic {
    static constexpr std::size_t outputDim = Dim;
    template <typename Output, typename A, typename B, typename C>
    XAD_HD void forward(Output& out, const A& a, const B& b, const C& c) const {
        for (std::size_t i = 0; i < Dim; ++i) out[i] = a[i] * b[i] + c[i];
    }
    template <typename Output, typename A, typename B, typename C>
    XAD_HD void backward(const Output& out, A& a, B& b, C& c) const {
        for (std::size_t i = 0; i < Dim; ++i) {
            a.add_grad(i, out.grad(i) * b[i]);
            b.add_grad(i, out.grad(i) * a[i]);
            c.add_grad(i, out.grad(i));
        }
    }
};

XAD_HD inline int run_case(int id, double* out) {
    int n = 0;
    auto put = [&](double v) { out[n++] = v; };
    switch (id) {
        case 0: {  // VariableRef on external buffers: tests/test_variable.cu:19-45, expectations :114-117
            float data[3], grad[3];
            VariableRef<3, float> var(data, grad);
            for (std::size_t i = 0; i < 3; ++i) var[i] = static_cast<float>(i + 1);
            var.zero_grad();
            for (std::size_t i = 0; i < 3; ++i) var.add_grad(i, static_cast<float>(i * 2));
            for (std::size_t i = 0; i < 3; ++i) put(var.data()[i]);
            for (std::size_t i = 0; i < 3; ++i) put(var.grad()[i]);
            var.zero_grad();  // :47-58, expectations :153-155
            for (std::size_t i = 0; i < 3; ++i) put(var.grad(i));
            break;
        }
        case 1: {  // Variable with its own storage: tests/test_variable.cu:61-78, expectations :173-180
            Variable<3, float> var;
            var.zero_grad();
            for (std::size_t i = 0; i < 3; ++i) {
                var[i] = static_cast<float>(i + 10);
                var.add_grad(i, static_cast<float>(i * 3));
            }
            for (std::size_t i = 0; i < 3; ++i) put(var[i]);
            for (std::size_t i = 0; i < 3; ++i) put(var.grad(i));
            auto view = var.ref();  // the view sees the same storage
            view.add_grad(1, 0.5f);
            put(var.grad(1));
            Variable<2, double> filled(7.5);
            const double src[2] = {1.25, -2.5};
            Variable<2, double> copied(src);
            put(filled[0]); put(filled[1]); put(copied[0]); put(copied[1]); put(copied.grad(0));
            break;
        }
        case 2: {  // DenseMatrix access and transpose: tests/test_dense_matrix.cu, tests/test_matrix_transpose.cu:124-133
            DenseMatrix<float, 2, 3> m;
            for (std::size_t r = 0; r < 2; ++r)
                for (std::size_t c = 0; c < 3; ++c) m(r, c) = static_cast<float>(r * 3 + c + 1);  // 1..6
            for (std::size_t i = 0; i < 6; ++i) put(m[i]);
            auto t = m.transpose();  // 3 x 2: 1 4 2 5 3 6
            for (std::size_t i = 0; i < 6; ++i) put(t[i]);
            m.add_grad(4, 2.0f);
            m.add_grad(4, 0.5f);
            put(m.grad(4));
            m.zero_grad();
            put(m.grad(4));
            break;
        }
        case 3: {  // dense x dense: [[1,2],[3,4]] [[5,6],[7,8]] = [[19,22],[43,50]]
            DenseMatrix<double, 2, 2> a, b;
            for (std::size_t i = 0; i < 4; ++i) {
                a[i] = static_cast<double>(i + 1);
                b[i] = static_cast<double>(i + 5);
            }
            auto c = a * b;
            for (std::size_t i = 0; i < 4; ++i) put(c[i]);
            auto d = a * b.transpose();  // [[17,23],[39,53]]
            for (std::size_t i = 0; i < 4; ++i) put(d[i]);
            break;
        }
        case 4: {  // DiagonalMatrixView: tests/test_diagonal_matrix.cu:22-91, expectations :119-127, :145-149, :167-171
            float data[3], grad[3];
            VariableRef<3, float> var(data, grad);
            DiagonalMatrixView<float, 3> diag(var);
            for (std::size_t i = 0; i < 3; ++i) diag[i] = static_cast<float>(i + 1);
            for (std::size_t i = 0; i < 3; ++i)
                for (std::size_t j = 0; j < 3; ++j) put(diag(i, j));
            DenseMatrix<float, 3, 2> tall;
            for (std::size_t i = 0; i < 6; ++i) tall[i] = static_cast<float>(i + 1);
            auto left = diag * tall;  // [1,2,6,8,15,18]
            for (std::size_t i = 0; i < 6; ++i) put(left[i]);
            DenseMatrix<float, 2, 3> wide;
            for (std::size_t i = 0; i < 6; ++i) wide[i] = static_cast<float>(i + 1);
            auto right = wide * diag;  // [1,4,9,4,10,18]
            for (std::size_t i = 0; i < 6; ++i) put(right[i]);
            auto same = diag.transpose();
            put(same(1, 1));
            Variable<2, double> own(3.0);
            auto view = make_diagonal_matrix_view(own);
            view.add_grad(1, 4.0);
            put(own.grad(1)); put(view(0, 1)); put(view(1, 1));
            break;
        }
        case 5: {  // SymmetricMatrixView: tests/test_symmetric_matrix.cu:21-100, expectations :130-139, :158-163, :182-192
            float data[6], grad[6];
            VariableRef<6, float> var(data, grad);
            auto sym = make_symmetric_matrix_view<3>(var);
            sym(0, 0) = 1; sym(0, 1) = 2; sym(0, 2) = 3; sym(1, 1) = 4; sym(1, 2) = 5; sym(2, 2) = 6;
            put(sym(0, 0)); put(sym(0, 1)); put(sym(1, 0)); put(sym(1, 1)); put(sym(2, 0)); put(sym(2, 2));
            put(sym(1, 0)); put(sym(2, 1));
            auto t = sym.transpose();
            put(t(0, 0)); put(t(0, 1)); put(t(1, 0)); put(t(1, 1)); put(t(2, 1)); put(t(1, 2));
            for (std::size_t i = 0; i < 6; ++i) put(sym[i]);  // storage order
            put(static_cast<double>(SymmetricMatrixView<float, 3, Variable<6, float>>::storage_size));
            put(static_cast<double>(SymmetricMatrixView<double, 4, Variable<10, double>>::storage_size));
            // symmetric x dense through the generic product: S [1,0,0]^T = first column
            DenseMatrix<float, 3, 1> e0;
            e0[0] = 1;
            auto col = sym * e0;
            put(col[0]); put(col[1]); put(col[2]);
            break;
        }
        case 6: {  // ConstArray arithmetic: tests/test_const_array.cu
            const float a_init[3] = {1.f, 2.f, 3.f}, b_init[3] = {4.f, 5.f, 6.f};
            ConstArray<float, 3> a(a_init), b(b_init);
            auto s = a + b, d = b - a, p = a * b, q = b / a;
            for (int i = 0; i < 3; ++i) put(s[i]);
            for (int i = 0; i < 3; ++i) put(d[i]);
            for (int i = 0; i < 3; ++i) put(p[i]);
            for (int i = 0; i < 3; ++i) put(q[i]);
            a += b;  // 5 7 9
            a *= b;  // 20 35 54
            a -= b;  // 16 30 48
            a /= b;  // 4 6 8
            for (int i = 0; i < 3; ++i) put(a[i]);
            // mixing with differentiable variables, the way a kernel accumulates a pixel
            // (examples/mini-gaussian-splatting/gaussian_splatting_kernel.cu:61, :100-104)
            Variable<3, float> v(2.0f);
            ConstArray<float, 3> pixel{};
            pixel += v;
            pixel += v;
            auto rest = b - v;   // ConstArray - Variable
            auto rest2 = v - b;  // Variable - ConstArray on plain values is not this overload: it builds a node
            rest2.forward();
            for (int i = 0; i < 3; ++i) put(pixel[i]);
            for (int i = 0; i < 3; ++i) put(rest[i]);
            for (int i = 0; i < 3; ++i) put(rest2[i]);
            const int ints[2] = {7, 9};
            ConstArray<int, 2> ia(ints);
            auto twice = ia + ia;
            put(twice[0]); put(twice[1]);
            break;
        }
        case 7: {  // scalar operators: tests/test_variable_operators.cu:94-101 (+2.5), :266-274, :339-347 (x1.5), :412-420 (/3)
            float data[3] = {1.f, 2.f, 3.f}, grad[3] = {0.f, 0.f, 0.f};
            VariableRef<3, float> x(data, grad);
            auto plus = x + 2.5f;
            plus.forward();
            for (std::size_t i = 0; i < 3; ++i) plus.add_grad(i, 1.0f);
            plus.backward();
            for (std::size_t i = 0; i < 3; ++i) put(plus[i]);
            for (std::size_t i = 0; i < 3; ++i) put(grad[i]);
            x.zero_grad();
            auto minus = x - 0.5f;
            minus.run();
            for (std::size_t i = 0; i < 3; ++i) put(minus[i]);
            for (std::size_t i = 0; i < 3; ++i) put(grad[i]);
            x.zero_grad();
            auto times = x * 1.5f;
            times.run();
            for (std::size_t i = 0; i < 3; ++i) put(times[i]);
            for (std::size_t i = 0; i < 3; ++i) put(grad[i]);
            x.zero_grad();
            auto over = x / 3.0f;
            over.run();
            for (std::size_t i = 0; i < 3; ++i) put(over[i]);
            for (std::size_t i = 0; i < 3; ++i) put(grad[i]);
            break;
        }
        case 8: {  // variable-variable operators: tests/operation/binary/test_variable_operators.cu:87-96
            Variable<2, double> a, b;
            a[0] = 2.0; a[1] = -3.0; b[0] = 4.0; b[1] = 0.5;
            auto s = a + b; s.run();
            put(s[0]); put(s[1]); put(a.grad(0)); put(b.grad(1));
            a.zero_grad(); b.zero_grad();
            auto d = a - b; d.run();
            put(d[0]); put(d[1]); put(a.grad(0)); put(b.grad(1));
            a.zero_grad(); b.zero_grad();
            auto p = a * b; p.run();
            put(p[0]); put(p[1]); put(a.grad(0)); put(a.grad(1)); put(b.grad(0)); put(b.grad(1));
            a.zero_grad(); b.zero_grad();
            auto q = a / b; q.run();
            put(q[0]); put(q[1]); put(a.grad(0)); put(a.grad(1)); put(b.grad(0)); put(b.grad(1));
            break;
        }
        case 9: {  // op::broadcast: tests/operation/unary/test_broadcast.cu:31-52 (sum 10, :110-119), :196-223 (:251-266)
            float in_data[1] = {3.5f}, in_grad[1] = {0.f};
            VariableRef<1, float> input(in_data, in_grad);
            input.zero_grad();
            auto wide = op::broadcast<4>(input);
            wide.forward();
            for (std::size_t i = 0; i < 4; ++i) put(wide[i]);
            for (std::size_t i = 0; i < 4; ++i) wide.add_grad(i, static_cast<float>(i + 1));
            wide.backward();
            put(in_grad[0]);
            float s_data[1] = {2.f}, s_grad[1] = {0.f}, v_data[3] = {1.f, 3.f, 5.f}, v_grad[3] = {0.f, 0.f, 0.f};
            VariableRef<1, float> scalar(s_data, s_grad);
            VariableRef<3, float> vector(v_data, v_grad);
            auto spread = op::broadcast<3>(scalar);
            auto result = spread + vector;
            result.forward();
            for (std::size_t i = 0; i < 3; ++i) put(result[i]);
            for (std::size_t i = 0; i < 3; ++i) result.add_grad(i, 1.0f);
            result.backward();
            put(s_grad[0]);
            for (std::size_t i = 0; i < 3; ++i) put(v_grad[i]);
            // the materialising form gives the same numbers
            Variable<1, double> one(1.5);
            auto copies = xyz_autodiff::broadcast<3>(one);
            copies.forward();
            for (std::size_t i = 0; i < 3; ++i) copies.add_grad(i, static_cast<double>(i + 1));
            copies.backward();
            put(copies[2]); put(one.grad(0));
            break;
        }
        case 10: {  // graphs with shared nodes: tests/test_dag_backward.cu:43-67 (=4), :90-117 (=4), :140-158 (=7)
            double a_data[1] = {1.0}, a_grad[1] = {0.0}, two[1] = {2.0}, two_g[1] = {0.0}, three[1] = {3.0}, three_g[1] = {0.0};
            {
                VariableRef<1, double> a(a_data, a_grad), c2(two, two_g), c3(three, three_g);
                auto b = op::add(a, c2);
                auto c = op::mul(a, c3);
                auto d = op::add(b, c);
                d.run();
                put(d[0]); put(a_grad[0]);
            }
            a_data[0] = 2.0; a_grad[0] = 0.0; two[0] = 2.0; three[0] = 1.0;
            {
                VariableRef<1, double> a(a_data, a_grad), c2(two, two_g), c1(three, three_g);
                auto b = op::mul(a, c2);
                auto c = op::add(a, c1);
                auto t = op::add(b, c);
                auto d = op::add(t, a);
                d.run();
                put(d[0]); put(a_grad[0]);
            }
            a_data[0] = 3.0; a_grad[0] = 0.0;
            {
                VariableRef<1, double> a(a_data, a_grad);
                auto b = op::mul(a, a);
                auto c = op::add(b, a);
                c.run();
                put(c[0]); put(a_grad[0]);
            }
            {  // DuplicateAddNetwork: tests/operation/base/test_linear_regression_network.cu:145-165 -> (2, 2)
                Variable<1, double> a(0.7), b(-1.3);
                auto ab = a + b;
                auto ab2 = a + b;
                auto sum = ab + ab2;
                sum.run();
                put(sum[0]); put(a.grad(0)); put(b.grad(0));
            }
            {  // an intermediate node with operation inputs, consumed twice:
               // y = l1(c2) + l2(c2), c2 = (a*b)*2.  d y / d a = 2 b (sign(c2) + c2/|c2|) = 4 b for positive a b.
                Variable<1, double> a(1.5), b(2.0);
                auto ab = a * b;
                auto c2 = ab * 2.0;
                auto n1 = op::l1_norm(c2);
                auto n2 = op::l2_norm(c2);
                auto y = n1 + n2;
                y.run();
                put(y[0]); put(a.grad(0)); put(b.grad(0));
                y.run();  // a second run of the same graph object starts from clean intermediate gradients
                put(a.grad(0));
            }
            break;
        }
        case 11: {  // chaining f = x z + y with an upstream gradient: tests/operation/base/test_operation_chaining.cu:33-50, :217-226
            double value[3] = {1.5, -0.5, 2.0}, grad[3] = {0.0, 0.0, 0.0};
            VariableRef<1, double> x(&value[0], &grad[0]), y(&value[1], &grad[1]), z(&value[2], &grad[2]);
            auto xz = op::mul(x, z);
            auto f = op::add(xz, y);
            f.forward();
            f.zero_grad();
            f.add_grad(0, 0.75);
            f.backward();
            put(f[0]); put(grad[0]); put(grad[1]); put(grad[2]);  // 0.75 * (z, 1, x)
            double ngrad[3] = {0.0, 0.0, 0.0};
            VariableRef<1, double> xn(&value[0], &ngrad[0]), yn(&value[1], &ngrad[1]), zn(&value[2], &ngrad[2]);
            auto xzn = op::mul(xn, zn);
            auto fn = op::add(xzn, yn);
            fn.forward();
            fn.zero_grad();
            fn.add_grad(0, 0.75);
            fn.backward_numerical(1e-7);
            put(ngrad[0]); put(ngrad[1]); put(ngrad[2]);
            break;
        }
        case 12: {  // a user-defined logic and a user-defined node inside library graphs
            Variable<2, double> x;
            x[0] = 1.0; x[1] = -2.0;
            UserShiftLogic<2> shift{0.25};
            UnaryOperation<2, UserShiftLogic<2>, Variable<2, double>> shifted(shift, x);
            auto sq = op::squared(shifted);
            auto total = op::sum(sq);
            total.run();
            put(total[0]); put(x.grad(0)); put(x.grad(1));  // sum (x + c)^2: 2 (x + c)
            x.zero_grad();
            auto ex = op::exp(x);
            UserDoubleNode<decltype(ex)> doubled(ex);  // foreign consumer of a library node
            auto s = op::sum(doubled);                 // library consumer of a foreign node
            s.run();
            put(s[0]); put(x.grad(0)); put(x.grad(1));  // 2 exp(x)
            break;
        }
        case 13: {  // math dispatcher, fp32: tests/test_math_dispatcher.cu:42-67
            const float x = 1.0f;
            put(math::exp(x)); put(math::log(math::exp(x))); put(math::sin(x)); put(math::cos(x)); put(math::tan(x));
            put(math::sinh(x)); put(math::cosh(x)); put(math::tanh(x)); put(math::sqrt(4.0f)); put(math::pow(2.0f, 3.0f));
            put(math::abs(-2.5f)); put(math::max(1.0f, 2.0f)); put(math::min(1.0f, 2.0f));
            put(math::sigmoid(0.0f)); put(math::relu(-1.0f)); put(math::relu(2.0f)); put(math::leaky_relu(-1.0f));
            put(math::elu(-1.0f)); put(math::softplus(0.0f)); put(math::swish(1.0f)); put(math::gelu(1.0f));
            float s, c;
            math::sincos(2.5f, s, c);
            put(s); put(c);
            break;
        }
        case 14: {  // math dispatcher, fp64: tests/test_math_dispatcher.cu:70-95
            const double x = 1.0;
            put(math::exp(x)); put(math::log(math::exp(x))); put(math::sin(x)); put(math::cos(x)); put(math::tan(x));
            put(math::sinh(x)); put(math::cosh(x)); put(math::tanh(x)); put(math::sqrt(4.0)); put(math::pow(2.0, 3.0));
            put(math::abs(-2.5)); put(math::max(1.0, 2.0)); put(math::min(1.0, 2.0));
            put(math::sigmoid(0.0)); put(math::relu(-1.0)); put(math::relu(2.0)); put(math::leaky_relu(-1.0));
            put(math::elu(-1.0)); put(math::softplus(0.0)); put(math::swish(1.0)); put(math::gelu(1.0));
            double s, c;
            math::sincos(2.5, s, c);
            put(s); put(c);
            break;
        }
        case 15: {  // the regression network written with operators, analytic and numerical:
                    // tests/operation/base/test_linear_regression_network.cu:39-78, parameter sets :186-196,
                    // :211-219, :282-290, :306-314 (a, b, c, d, x1, x2, y_target)
            const double sets[4][7] = {{1.0, 1.5, 0.5, 0.2, 2.0, 1.5, 3.0},
                                       {0.8, 1.2, -0.3, 0.5, 1.0, 0.8, 2.5},
                                       {10.0, 15.0, -8.0, 5.0, 20.0, -10.0, 100.0},
                                       {0.001, 0.002, -0.001, 0.0001, 0.01, -0.01, 0.001}};
            for (int k = 0; k < 4; ++k) {
                for (int numerical = 0; numerical < 2; ++numerical) {
                    double value[4] = {sets[k][0], sets[k][1], sets[k][2], sets[k][3]}, diff[4] = {0.0, 0.0, 0.0, 0.0};
                    VariableRef<1, double> a_var(&value[0], &diff[0]), b_var(&value[1], &diff[1]), c_var(&value[2], &diff[2]),
                        d_var(&value[3], &diff[3]);
                    auto x1_minus_a = a_var - sets[k][4];
                    auto x1_term = op::squared(x1_minus_a);
                    auto x2_minus_c = c_var - sets[k][5];
                    auto x2_squared = op::squared(x2_minus_c);
                    auto x2_term = b_var * x2_squared;
                    auto combined_terms = x1_term + x2_term;
                    auto y_pred = combined_terms + d_var;
                    auto y_diff = y_pred - sets[k][6];
                    auto loss = op::squared(y_diff);
                    if (numerical)
                        loss.run_numerical(k == 3 ? 1e-8 : (k == 2 ? 1e-5 : 1e-6));
                    else
                        loss.run();
                    if (!numerical) put(loss[0]);
                    for (int j = 0; j < 4; ++j) put(diff[j]);
                }
            }
            break;
        }
        case 16: {  // TernaryOperation (operation.cuh:382-623 of the reference) with a user logic, y = a b + c
            using V2 = Variable<2, double>;
            UserMulAddLogic<2> fma_logic;
            {   // three leaves: values, analytic gradients, then the numerical ones
                V2 a, b, c;
                a[0] = 1.5; a[1] = -2.0; b[0] = 0.5; b[1] = 3.0; c[0] = 0.25; c[1] = -1.0;
                TernaryOperation<2, UserMulAddLogic<2>, V2, V2, V2> y(fma_logic, a, b, c);
                y.run();
                put(y[0]); put(y[1]);
                put(a.grad(0)); put(a.grad(1)); put(b.grad(0)); put(b.grad(1)); put(c.grad(0)); put(c.grad(1));
                a.zero_grad(); b.zero_grad(); c.zero_grad();
                y.run_numerical(1e-6);
                put(a.grad(0)); put(a.grad(1)); put(b.grad(0)); put(b.grad(1)); put(c.grad(0)); put(c.grad(1));
            }
            {   // operands that are nodes, one of them in two slots: y = e * e + n, e = exp(x), n = -x
                //   d y / d x = 2 e^2x - 1
                Variable<1, double> x(0.3);
                auto e = op::exp(x);
                auto n = op::neg(x);
                UserMulAddLogic<1> fma1;
                TernaryOperation<1, UserMulAddLogic<1>, decltype(e), decltype(e), decltype(n)> y(fma1, e, e, n);
                y.run();
                put(y[0]); put(x.grad(0));
            }
            {   // a ternary node consumed twice: z = y + y^2 with y = a b + c (3.5): d z / d y = 1 + 2 y = 8
                Variable<1, double> a(2.0), b(1.5), c(0.5);
                UserMulAddLogic<1> fma1;
                TernaryOperation<1, UserMulAddLogic<1>, Variable<1, double>, Variable<1, double>, Variable<1, double>> y(fma1, a, b, c);
                auto y2 = op::squared(y);
                auto z = y + y2;
                z.run();
                put(z[0]); put(a.grad(0)); put(b.grad(0)); put(c.grad(0));
            }
            break;
        }
        case 17: {  // several roots over one shared node, and forward passes that no backward follows
            {   // s = exp(x); r1 = -s, r2 = s^2; forward both, seed both, backward both:
                //   d (r1 + r2) / d x = (2 s - 1) s   (the counts of operation.cuh:53-83 of the reference)
                Variable<1, double> x(0.5);
                auto s = op::exp(x);
                auto r1 = op::neg(s);
                auto r2 = op::squared(s);
                r1.forward();
                r2.forward();
                r1.add_grad(0, 1.0);
                r2.add_grad(0, 1.0);
                r1.backward();
                put(x.grad(0));  // s has one more consumer to hear from: nothing has reached x yet
                r2.backward();
                put(r1[0]); put(r2[0]); put(x.grad(0));
            }
            {   // forward twice, then backward: the first pass leaves nothing behind
                Variable<1, double> x(0.5);
                auto s = op::exp(x);
                auto r = op::squared(s);
                r.forward();
                x[0] = 0.25;  // and the second pass sees the new value
                r.forward();
                r.add_grad(0, 1.0);
                r.backward();
                put(r[0]); put(x.grad(0));  // e^0.5, 2 e^0.5
            }
            {   // a root forwarded and abandoned does not disturb another root over the same node
                Variable<1, double> x(0.5);
                auto s = op::exp(x);
                auto abandoned = op::neg(s);
                auto r = op::squared(s);
                abandoned.forward();
                abandoned.forward();  // takes back its own visit first: s still has exactly one
                r.run();
                put(x.grad(0));  // s waits for `abandoned`: nothing yet
                abandoned.add_grad(0, 1.0);
                abandoned.backward();
                put(x.grad(0));  // (2 s - 1) s
            }
            {   // a node with two consumers inside one graph, walked twice before the backward pass:
                //   y = s + s^2 through a broadcast, s = exp(x); the second walk sees x = 0.25 and counts nothing twice
                Variable<1, double> x(0.5);
                auto s = op::exp(x);
                auto s2 = op::squared(s);
                auto y = s + s2;
                auto wide = op::broadcast<3>(y);
                auto total = op::sum(wide);
                total.forward();
                put(total[0]);  // 3 (e^0.5 + e)
                x[0] = 0.25;
                total.forward();
                total.add_grad(0, 1.0);
                total.backward();
                put(total[0]); put(x.grad(0));  // 3 (e^0.25 + e^0.5), 3 (e^0.25 + 2 e^0.5)
            }
            break;
        }
        default:
            return -1;
    }
    return n;
}

}  // namespace xad_test
