// Factories of rt::Node.  Field packing follows src/runtime/node.cu:56-598 so that a node built
// here is byte-for-byte what the reference's operator graph hands to a kernel table.
#include "node.hh"

#include <algorithm>

namespace rt
{

const char* Node::OP_NAMES[Node::OP_COUNT] = {
    "mat_mat_mul", "mat_rvect_add", "sigmoid", "mse", "softmax", "log_softmax", "softmax_cross_entropy",
    "conv2d", "relu", "relu_leaky", "tanh", "mse_grad", "sigmoid_grad", "mat_mul_add", "tmat_mat_mul",
    "mat_tmat_mul", "mat_sum_rows", "mat_sum_cols", "softmax_cross_entropy_grad", "relu_grad",
    "conv2d_bias_add", "update", "sigmoid_cross_entropy", "sigmoid_cross_entropy_grad", "conv2d_input_grad",
    "conv2d_kernel_grad", "argmax_acc", "moment_update", "moment_update2", "adam_update", "leaky_relu_grad",
    "conv2d_bias_add_grad", "tanh_grad", "conv2d_transpose", "conv2d_transpose_input_grad",
    "conv2d_transpose_kernel_grad", "add"};

const char* Node::name_of(int type)
{
    if (type == OP_NOP)
        return "nop";
    return type >= 0 && type < OP_COUNT ? OP_NAMES[type] : "?";
}

Node::Node(int type_, std::vector<Node*> preds_)
    : type(type_), use_simd(false), in1(nullptr), in2(nullptr), in3(nullptr), out1(nullptr), out2(nullptr),
      cons1(0), cons2(0), cons3(0), cons4(0), len1(0), len2(0), len3(0), intconst{0, 0}, intconst2{0, 0},
      sizes1{0, 0, 0, 0}, sizes2{0, 0, 0, 0}, sizes3{0, 0, 0, 0}, int_cons1(0), int_cons2(0), alpha_leaky(0)
{
    // null predecessors (inputs and variables have no node) are dropped, src/runtime/node.cu:613-620
    for (Node* n : preds_)
        if (n)
        {
            n->succs.push_back(this);
            preds.push_back(n);
        }
}

namespace
{
// Small fluent helper so that each factory below is one expression.
struct Fill
{
    Node* n;
    Fill(int type, const Node::Preds& preds) : n(new Node(type, preds)) {}
    Fill& in(const dbl_t* a, const dbl_t* b = nullptr, const dbl_t* c = nullptr) { n->in1 = a; n->in2 = b; n->in3 = c; return *this; }
    Fill& out(dbl_t* a, dbl_t* b = nullptr) { n->out1 = a; n->out2 = b; return *this; }
    Fill& len(std::size_t a, std::size_t b = 0, std::size_t c = 0) { n->len1 = a; n->len2 = b; n->len3 = c; return *this; }
    Fill& cons(dbl_t a, dbl_t b = 0, dbl_t c = 0, dbl_t d = 0) { n->cons1 = a; n->cons2 = b; n->cons3 = c; n->cons4 = d; return *this; }
    Fill& i2(int (Node::*field)[2], const int v[]) { std::copy(v, v + 2, n->*field); return *this; }
    Fill& i4(int (Node::*field)[4], const int v[]) { std::copy(v, v + 4, n->*field); return *this; }
    operator Node*() const { return n; }
};
}  // namespace

Node* Node::nop(const Preds& preds) { return new Node(OP_NOP, preds); }

Node* Node::op_conv2d(const dbl_t* input, const dbl_t* kernel, const int strides[], int pad_top, int pad_left,
                      dbl_t* output, const int input_size[], const int kernel_size[], const Preds& preds)
{
    Node* n = Fill(OP_CONV2D, preds).in(input, kernel).out(output).i2(&Node::intconst, strides)
                  .i4(&Node::sizes1, input_size).i4(&Node::sizes2, kernel_size);
    n->int_cons1 = pad_top;
    n->int_cons2 = pad_left;
    return n;
}

Node* Node::op_conv2d_bias_add(const dbl_t* z, const dbl_t* bias, dbl_t* output, const int input_size[],
                               const Preds& preds)
{
    return Fill(OP_CONV2D_BIAS_ADD, preds).in(z, bias).out(output).i4(&Node::sizes1, input_size);
}

Node* Node::op_conv2d_bias_add_grad(const dbl_t* z, const int size[], dbl_t* output, const Preds& preds)
{
    return Fill(OP_CONV2D_BIAS_ADD_GRAD, preds).in(z).out(output).i4(&Node::sizes1, size);
}

Node* Node::op_conv2d_input_grad(const dbl_t* y, const dbl_t* kernel, const int strides[], dbl_t* output,
                                 const int y_size[], const int kernel_size[], const int input_size[],
                                 const Preds& preds)
{
    // intconst2 = spatial extent of the input, i.e. input_size[1..2]
    return Fill(OP_CONV2D_INPUT_GRAD, preds).in(y, kernel).out(output).i2(&Node::intconst, strides)
        .i2(&Node::intconst2, input_size + 1).i4(&Node::sizes1, y_size).i4(&Node::sizes2, kernel_size);
}

Node* Node::op_conv2d_kernel_grad(const dbl_t* y, const dbl_t* input, const int strides[], dbl_t* output,
                                  const int y_size[], const int input_size[], const int padded_size[],
                                  const Preds& preds)
{
    return Fill(OP_CONV2D_KERNEL_GRAD, preds).in(y, input).out(output).i2(&Node::intconst, strides)
        .i2(&Node::intconst2, padded_size).i4(&Node::sizes1, y_size).i4(&Node::sizes2, input_size);
}

Node* Node::op_conv2d_transpose(const dbl_t* input, const dbl_t* kernel, const int out_size[], const int strides[],
                                dbl_t* output, const int input_size[], const int kernel_size[], const Preds& preds)
{
    return Fill(OP_CONV2D_TRANSPOSE, preds).in(input, kernel).out(output).i2(&Node::intconst, strides)
        .i4(&Node::sizes1, out_size).i4(&Node::sizes2, input_size).i4(&Node::sizes3, kernel_size);
}

Node* Node::op_conv2d_transpose_input_grad(const dbl_t* y, const dbl_t* kernel, const int strides[], dbl_t* output,
                                           const int y_size[], const int kernel_size[], const int input_size[],
                                           const Preds& preds)
{
    return Fill(OP_CONV2D_TRANSPOSE_INPUT_GRAD, preds).in(y, kernel).out(output).i2(&Node::intconst, strides)
        .i2(&Node::intconst2, input_size + 1).i4(&Node::sizes1, y_size).i4(&Node::sizes2, kernel_size);
}

Node* Node::op_conv2d_transpose_kernel_grad(const dbl_t* y, const dbl_t* input, const int strides[], dbl_t* output,
                                            const int y_size[], const int input_size[], const int kernel_size[],
                                            const Preds& preds)
{
    return Fill(OP_CONV2D_TRANSPOSE_KERNEL_GRAD, preds).in(y, input).out(output).i2(&Node::intconst, strides)
        .i4(&Node::sizes1, y_size).i4(&Node::sizes2, input_size).i4(&Node::sizes3, kernel_size);
}

Node* Node::op_mat_mat_mul(const dbl_t* left, const dbl_t* right, dbl_t* output, std::size_t rowsl,
                           std::size_t colsl, std::size_t colsr, const Preds& preds)
{
    return Fill(OP_MAT_MAT_MUL, preds).in(left, right).out(output).len(rowsl, colsl, colsr);
}

Node* Node::op_mat_mul_add(const dbl_t* x, const dbl_t* w, const dbl_t* b, dbl_t* output, std::size_t rowsx,
                           std::size_t colsx, std::size_t colsw, const Preds& preds)
{
    return Fill(OP_MAT_MUL_ADD, preds).in(x, w, b).out(output).len(rowsx, colsx, colsw);
}

Node* Node::op_tmat_mat_mul(const dbl_t* left, const dbl_t* right, dbl_t* output, std::size_t rowsl,
                            std::size_t colsl, std::size_t colsr, const Preds& preds)
{
    return Fill(OP_TMAT_MAT_MUL, preds).in(left, right).out(output).len(rowsl, colsl, colsr);
}

Node* Node::op_mat_tmat_mul(const dbl_t* left, const dbl_t* right, dbl_t* output, std::size_t rowsl,
                            std::size_t colsl, std::size_t colsr, const Preds& preds)
{
    return Fill(OP_MAT_TMAT_MUL, preds).in(left, right).out(output).len(rowsl, colsl, colsr);
}

Node* Node::op_mat_rvect_add(const dbl_t* left, const dbl_t* right, dbl_t* output, std::size_t rows,
                             std::size_t cols, const Preds& preds)
{
    return Fill(OP_MAT_RVECT_ADD, preds).in(left, right).out(output).len(rows, cols);
}

Node* Node::op_mat_sum_rows(const dbl_t* arg, dbl_t* out, std::size_t rows, std::size_t cols, const Preds& preds)
{
    return Fill(OP_MAT_SUM_ROWS, preds).in(arg).out(out).len(rows, cols);
}

Node* Node::op_mat_sum_cols(const dbl_t* arg, dbl_t* out, std::size_t rows, std::size_t cols, const Preds& preds)
{
    return Fill(OP_MAT_SUM_COLS, preds).in(arg).out(out).len(rows, cols);
}

Node* Node::op_relu(const dbl_t* args, dbl_t* out, std::size_t len, const Preds& preds)
{
    return Fill(OP_RELU, preds).in(args).out(out).len(len);
}

Node* Node::op_relu_leaky(const dbl_t* args, dbl_t* out, std::size_t len, const dbl_t alpha, const Preds& preds)
{
    Node* n = Fill(OP_RELU_LEAKY, preds).in(args).out(out).len(len);
    n->alpha_leaky = alpha;
    return n;
}

Node* Node::op_sigmoid(const dbl_t* args, dbl_t* out, std::size_t len, const Preds& preds)
{
    return Fill(OP_SIGMOID, preds).in(args).out(out).len(len);
}

Node* Node::op_tanh(const dbl_t* args, dbl_t* out, std::size_t len, const Preds& preds)
{
    return Fill(OP_TANH, preds).in(args).out(out).len(len);
}

Node* Node::op_relu_grad(const dbl_t* z, const dbl_t* dout, dbl_t* out, std::size_t len, const Preds& preds)
{
    return Fill(OP_RELU_GRAD, preds).in(z, dout).out(out).len(len);
}

Node* Node::op_leaky_relu_grad(const dbl_t* z, const dbl_t* dout, dbl_t* out, dbl_t alpha, std::size_t len,
                               const Preds& preds)
{
    return Fill(OP_LEAKY_RELU_GRAD, preds).in(z, dout).out(out).len(len).cons(alpha);
}

Node* Node::op_sigmoid_grad(const dbl_t* sig_out, const dbl_t* dout, dbl_t* out, std::size_t len, const Preds& preds)
{
    return Fill(OP_SIGMOID_GRAD, preds).in(sig_out, dout).out(out).len(len);
}

Node* Node::op_tanh_grad(const dbl_t* tanh_out, const dbl_t* dout, dbl_t* out, std::size_t len, const Preds& preds)
{
    return Fill(OP_TANH_GRAD, preds).in(tanh_out, dout).out(out).len(len);
}

Node* Node::op_add(const dbl_t* a, const dbl_t* b, dbl_t* out, std::size_t len, const Preds& preds)
{
    return Fill(OP_ADD, preds).in(a, b).out(out).len(len);
}

Node* Node::op_mse(const dbl_t* y, const dbl_t* y_hat, dbl_t* out, std::size_t rows, std::size_t cols,
                   const Preds& preds)
{
    return Fill(OP_MSE, preds).in(y, y_hat).out(out).len(rows, cols);
}

Node* Node::op_mse_grad(const dbl_t* y, const dbl_t* y_hat, dbl_t* out, std::size_t len, const Preds& preds)
{
    return Fill(OP_MSE_GRAD, preds).in(y, y_hat).out(out).len(len);
}

Node* Node::op_softmax(const dbl_t* args, dbl_t* out, std::size_t rows, std::size_t cols, const Preds& preds)
{
    return Fill(OP_SOFTMAX, preds).in(args).out(out).len(rows, cols);
}

Node* Node::op_log_softmax(const dbl_t* args, dbl_t* out, std::size_t rows, std::size_t cols, const Preds& preds)
{
    return Fill(OP_LOG_SOFTMAX, preds).in(args).out(out).len(rows, cols);
}

Node* Node::op_softmax_cross_entropy(const dbl_t* y, const dbl_t* logits, dbl_t* out, std::size_t rows,
                                     std::size_t cols, const Preds& preds)
{
    return Fill(OP_SOFTMAX_CROSS_ENTROPY, preds).in(y, logits).out(out).len(rows, cols);
}

Node* Node::op_softmax_cross_entropy_grad(const dbl_t* y, const dbl_t* logits, dbl_t* out, std::size_t rows,
                                          std::size_t cols, const Preds& preds)
{
    return Fill(OP_SOFTMAX_CROSS_ENTROPY_GRAD, preds).in(y, logits).out(out).len(rows, cols);
}

Node* Node::op_sigmoid_cross_entropy(const dbl_t* y, const dbl_t* logits, dbl_t* out, std::size_t len,
                                     const Preds& preds)
{
    return Fill(OP_SIGMOID_CROSS_ENTROPY, preds).in(y, logits).out(out).len(len);
}

Node* Node::op_sigmoid_cross_entropy_grad(const dbl_t* y, const dbl_t* logits, dbl_t* out, std::size_t len,
                                          const Preds& preds)
{
    return Fill(OP_SIGMOID_CROSS_ENTROPY_GRAD, preds).in(y, logits).out(out).len(len);
}

Node* Node::op_argmax_acc(const dbl_t* y, const dbl_t* y_hat, dbl_t* out, std::size_t rows, std::size_t cols,
                          const Preds& preds)
{
    return Fill(OP_ARGMAX_ACC, preds).in(y, y_hat).out(out).len(rows, cols);
}

Node* Node::op_update(dbl_t* var, const dbl_t* dt, const dbl_t* coeff, std::size_t len, const Preds& preds)
{
    return Fill(OP_UPDATE, preds).in(dt, coeff).out(var).len(len);
}

Node* Node::op_moment_update(dbl_t* var, const dbl_t* dt, dbl_t coeff1, dbl_t coeff2, std::size_t len,
                             const Preds& preds)
{
    return Fill(OP_MOMENT_UPDATE, preds).in(dt).out(var).len(len).cons(coeff1, coeff2);
}

Node* Node::op_moment_update2(dbl_t* var, const dbl_t* dt, dbl_t coeff1, dbl_t coeff2, std::size_t len,
                              const Preds& preds)
{
    return Fill(OP_MOMENT_UPDATE2, preds).in(dt).out(var).len(len).cons(coeff1, coeff2);
}

Node* Node::op_adam_update(dbl_t* var, dbl_t* t, const dbl_t* m, const dbl_t* v, dbl_t lr, dbl_t beta1, dbl_t beta2,
                           dbl_t eps, std::size_t len, const Preds& preds)
{
    return Fill(OP_ADAM_UPDATE, preds).in(m, v).out(var, t).len(len).cons(lr, beta1, beta2, eps);
}

}  // namespace rt
