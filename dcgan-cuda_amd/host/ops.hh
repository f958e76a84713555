// Operator graph with reverse-mode differentiation: the API that model code is written against
// (reference: src/ops -- OpsBuilder src/ops/ops-builder.hh:22-61, Op src/ops/op.hh:11-70,
// Graph src/ops/graph.hh:65-121, Shape src/ops/shape.hh:9-38, CompiledOp
// src/ops/compiled-op.hh:12-53).  Method names, argument meaning and error behaviour
// (std::runtime_error) are the reference's; the implementation is not: operators are one class
// parameterised by two closures (lowering to rt::Node instructions, and the chain rule), the
// execution order of a run is computed once per set of requested operators and cached, and
// tensors come from memory.hh.
#pragma once

#include <functional>
#include <iosfwd>
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "rt_graph.hh"
#include "types.hh"

namespace ops
{

class Shape
{
public:
    Shape(const std::vector<int>& dims = {}) : dims_(dims) {}
    const std::vector<int>& dims() const { return dims_; }
    std::size_t ndims() const { return dims_.size(); }
    int operator[](std::size_t i) const { return dims_.at(i); }
    bool defined() const;    // no -1 extent
    int total() const;       // product of the extents
    Shape transpose() const; // matrices only

private:
    std::vector<int> dims_;
};

bool operator==(const Shape& a, const Shape& b);
bool operator!=(const Shape& a, const Shape& b);
std::ostream& operator<<(std::ostream& os, const Shape& s);

class Op;

// What lowering an operator produced: its instructions, the tensors it owns (freed with it), and
// where its result lives.
struct CompiledOp
{
    Op* op = nullptr;
    std::vector<rt::Node*> nodes;
    std::vector<dbl_t*> tensors;
    rt::Node* out_node = nullptr;
    Shape out_shape;
    dbl_t* out_data = nullptr;
};

class Op
{
public:
    using CompileFn = std::function<void(Op&)>;
    using GradFn = std::function<Op*(Op&, std::size_t index, Op* dout)>;

    Op(const std::string& name, const Shape& shape, const std::vector<Op*>& preds = {});
    virtual ~Op() = default;

    const std::string& name_get() const { return name_; }
    void extend_name(const std::string& str) { name_ += ":" + str; }
    const Shape& shape_get() const { return shape_; }
    const std::vector<Op*>& preds() const { return preds_; }
    const std::vector<Op*>& succs() const { return succs_; }

    // Allocate the result and emit the rt::Node instructions (through Graph::add_compiled).
    virtual void compile();
    // Position of `pred` among the operands, or std::size_t(-1).
    std::size_t pred_index(const Op* pred) const;
    // The consumer of this operator through which `node` is reached (nullptr if none) / all of them.
    Op* pred_of(const Op* node);
    std::vector<Op*> preds_of(const Op* node);
    // d(C)/d(operand index) given dout = d(C)/d(this); dout == nullptr when C is this operator.
    virtual Op* child_grad(std::size_t index, Op* dout);

    CompileFn compile_fn;
    GradFn grad_fn;

private:
    friend class Graph;
    std::string name_;
    Shape shape_;
    std::vector<Op*> preds_;
    std::vector<Op*> succs_;
};

class Input : public Op
{
public:
    explicit Input(const Shape& shape);
    void compile() override;
};

class Variable : public Op
{
public:
    Variable(const Shape& shape, bool trainable);
    ~Variable() override;
    void compile() override;
    bool is_trainable() const { return trainable_; }
    dbl_t* data_begin() { return data_; }
    dbl_t* data_end() { return data_ + shape_get().total(); }
    void write(const dbl_t* host);
    void read(dbl_t* host) const;

private:
    dbl_t* data_;
    bool trainable_;
};

// Every other operator is a plain Op; the names below keep reference-style code compiling.
using Add = Op; using AdamUpdate = Op; using ArgmaxAccuracy = Op; using Conv2D = Op; using Conv2DBiasAdd = Op;
using Conv2DBiasAddGrad = Op; using Conv2DInputGrad = Op; using Conv2DKernelGrad = Op; using Conv2DTranspose = Op;
using Conv2DTransposeInputGrad = Op; using Conv2DTransposeKernelGrad = Op; using LeakyReluGrad = Op;
using MatMatMul = Op; using MatMulAdd = Op; using MatRvectAdd = Op; using MatSum = Op; using MomentUpdate = Op;
using MSE = Op; using MSEGrad = Op; using ReluGrad = Op; using Seq = Op; using SigmoidCrossEntropy = Op;
using SigmoidCrossEntropyGrad = Op; using SigmoidGrad = Op; using TanhGrad = Op; using Update = Op;
using VectSigmoid = Op; using VectRelu = Op; using VectReluLeaky = Op; using VectTanh = Op; using Reshape = Op;

class Graph
{
public:
    static Graph& instance();
    Graph(const Graph&) = delete;
    Graph& operator=(const Graph&) = delete;
    ~Graph();

    const std::vector<Op*>& ops_list() const { return ops_; }
    // Trainable variables `cost` depends on (all trainable variables if cost is nullptr).
    std::vector<Variable*> train_vars_get(Op* cost);

    void add(Op* op);            // takes ownership
    void add_var(Variable* var);

    // Evaluate `ops`.  `inputs` maps each Input to (host data, shape); outputs[i] receives the
    // result of ops[i] unless it is nullptr.  Operators are lowered on first use and re-lowered
    // when an input changes shape; inputs are copied in, the instruction list runs on the backend
    // program_mode() selects, outputs are copied out (src/ops/graph.cu:98-223).
    void run(std::vector<Op*> ops, const std::map<Input*, std::pair<const dbl_t*, Shape>>& inputs = {},
             const std::vector<dbl_t*>& outputs = {});

    void add_compiled(Op* op, const std::vector<rt::Node*> nodes, std::vector<dbl_t*> tensors, rt::Node* out_node,
                      const Shape& out_shape, dbl_t* out_data);
    const CompiledOp& compiled(Op* op);
    bool is_compiled(Op* op) const { return compiled_ops_.count(op) != 0; }

    // d(out)/d(var) as a graph operator (memoised); builds the intermediate gradient operators by
    // backpropagation (src/ops/graph.cu:243-324).
    Op* gradient(Op* out, Op* var);

    void debug_set(bool debug) { debug_ = debug; }
    // Off: run() hands the backend nothing but the instruction list, as src/ops/graph.cu:194-200 does
    // (hip::protect_all_tensors: every intermediate result is kept).  On (default): run() names the
    // tensors it reads back (hip::set_protected_tensors) and the backend may leave the others out.
    void name_results_set(bool on) { name_results_ = on; }
    // Trainable variables, in creation order, to / from a file: numpy's .npz when the path ends in
    // ".npz" (arrays arr_0, arr_1, ...), else a `DGV1` header followed per variable by the element
    // count and the fp32 data.
    void save_vars(const std::string& path);
    void load_vars(const std::string& path);
    // All variables (optimiser moments included) and the Adam step counters, as .npz.
    void save_state(const std::string& path);
    void load_state(const std::string& path);
    void add_counter(std::shared_ptr<dbl_t> t) { counters_.push_back(std::move(t)); }
    // Free every operator, tensor and instruction (end of program, or between tests).
    void exit_graph();

    // The instruction list the last run() executed (debugging and tests).
    const std::vector<rt::Node*>& last_schedule() const { return last_schedule_; }

private:
    Graph() = default;
    void compile_(Op* node);
    void remove_compiled_rec_(Op* op);
    Op* compute_gradient_(Op* out, Op* var);

    std::vector<Op*> ops_;
    std::vector<Variable*> vars_;
    std::vector<std::shared_ptr<dbl_t>> counters_;   // step counters of the Adam operators, creation order
    std::map<Input*, Shape> input_shapes_;
    std::map<Op*, CompiledOp> compiled_ops_;
    std::map<std::pair<Op*, Op*>, Op*> grads_;
    std::map<std::vector<Op*>, std::vector<rt::Node*>> schedules_;
    std::vector<rt::Node*> last_schedule_;
    rt::Graph* full_rt_graph_ = new rt::Graph;
    bool debug_ = false;
    bool name_results_ = true;
};

class OpsBuilder
{
public:
    static OpsBuilder& instance();
    OpsBuilder(const OpsBuilder&) = delete;
    OpsBuilder& operator=(const OpsBuilder&) = delete;

    Add* add(Op* left, Op* right);
    AdamUpdate* adam_update(Variable* var, Op* m, Op* v, dbl_t learning_rate, dbl_t beta1, dbl_t beta2, dbl_t eps);
    ArgmaxAccuracy* argmax_accuracy(Op* y, Op* y_hat);
    Conv2D* conv2d(Op* input, Op* kernel, const int* strides);
    Conv2DBiasAdd* conv2d_bias_add(Op* z, Op* bias);
    Conv2DBiasAddGrad* conv2d_bias_add_grad(Op* z);
    Conv2DInputGrad* conv2d_input_grad(Op* y, Op* kernel, const int* strides, const int* input_size);
    Conv2DKernelGrad* conv2d_kernel_grad(Op* y, Op* input, const int* strides, const int* kernel_size,
                                         const int* padded_size);
    Conv2DTranspose* conv2d_transpose(Op* input, Op* kernel, const int* out_size, const int* strides);
    Conv2DTransposeInputGrad* conv2d_transpose_input_grad(Op* y, Op* kernel, const int* strides,
                                                          const int* input_size);
    Conv2DTransposeKernelGrad* conv2d_transpose_kernel_grad(Op* y, Op* input, const int* strides,
                                                            const int* kernel_size);
    Input* input(const Shape& shape);
    LeakyReluGrad* leaky_relu_grad(Op* z, Op* dout, dbl_t alpha);
    MatMatMul* mat_mat_mul(Op* left, Op* right, bool left_tr = false, bool right_tr = false);
    MatMulAdd* mat_mul_add(Op* x, Op* w, Op* b);
    MatRvectAdd* mat_rvect_add(Op* left, Op* right);
    MatSum* mat_sum(Op* arg, std::size_t axis);
    MomentUpdate* moment_update(Variable* var, Op* dt, dbl_t coeff1, dbl_t coeff2, bool sq_update);
    MSE* mse(Op* y, Op* y_hat);
    MSEGrad* mse_grad(Op* y, Op* y_hat);
    ReluGrad* relu_grad(Op* z, Op* dout);
    Seq* seq(const std::vector<Op*>& ops);
    SigmoidCrossEntropy* sigmoid_cross_entropy(Op* y, Op* logits);
    SigmoidCrossEntropyGrad* sigmoid_cross_entropy_grad(Op* y, Op* logits);
    SigmoidGrad* sigmoid_grad(Op* sig_out, Op* dout);
    TanhGrad* tanh_grad(Op* tanh_out, Op* dout);
    Update* update(Variable* var, Op* dt, Op* coeff);
    Variable* variable(const Shape& shape, bool trainable = false);
    VectSigmoid* vect_sigmoid(Op* arg);
    VectRelu* vect_relu(Op* arg);
    VectReluLeaky* vect_relu_leaky(Op* arg, const dbl_t alpha = 0.2);
    VectTanh* vect_tanh(Op* arg);
    Reshape* reshape(Op* arg, const Shape& shape);

private:
    OpsBuilder() = default;
};

}  // namespace ops
