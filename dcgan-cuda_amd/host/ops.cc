#include "ops.hh"

#include <cstdlib>
#include <cstring>
#include "npz.hh"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <iostream>
#include <memory>
#include <set>
#include <stdexcept>

#include "backend.hh"
#include "memory.hh"

namespace ops
{

// ---- Shape -----------------------------------------------------------------------------------------
bool Shape::defined() const
{
    return std::find(dims_.begin(), dims_.end(), -1) == dims_.end();
}

int Shape::total() const
{
    int res = 1;
    for (int d : dims_)
        res *= d;
    return res;
}

Shape Shape::transpose() const
{
    if (dims_.size() != 2)
        throw std::runtime_error("Shape::transpose: not a matrix");
    return Shape({dims_[1], dims_[0]});
}

bool operator==(const Shape& a, const Shape& b) { return a.dims() == b.dims(); }
bool operator!=(const Shape& a, const Shape& b) { return !(a == b); }

std::ostream& operator<<(std::ostream& os, const Shape& s)
{
    os << '(';
    for (std::size_t i = 0; i < s.ndims(); ++i)
        os << (i ? ", " : "") << s[i];
    return os << ')';
}

// ---- Op --------------------------------------------------------------------------------------------
Op::Op(const std::string& name, const Shape& shape, const std::vector<Op*>& preds)
    : name_(name), shape_(shape), preds_(preds)
{
    for (Op* p : preds_)
        p->succs_.push_back(this);
}

void Op::compile()
{
    if (!compile_fn)
        throw std::runtime_error("operator '" + name_ + "' cannot be lowered");
    compile_fn(*this);
}

std::size_t Op::pred_index(const Op* pred) const
{
    auto it = std::find(preds_.begin(), preds_.end(), pred);
    return it == preds_.end() ? std::size_t(-1) : std::size_t(it - preds_.begin());
}

Op* Op::pred_of(const Op* node)
{
    for (Op* s : succs_)
        if (s == node || s->pred_of(node))
            return s;
    return nullptr;
}

std::vector<Op*> Op::preds_of(const Op* node)
{
    std::vector<Op*> res;
    for (Op* s : succs_)
        if (s == node || s->pred_of(node))
            res.push_back(s);
    return res;
}

Op* Op::child_grad(std::size_t index, Op* dout)
{
    if (!grad_fn)
        throw std::runtime_error("It's not possible to compute the gradient of this node");
    return grad_fn(*this, index, dout);
}

// ---- Input / Variable ------------------------------------------------------------------------------
Input::Input(const Shape& shape) : Op("input", shape) {}

void Input::compile()
{
    // the shape of an input is the one of the data bound to it by Graph::run
    throw std::logic_error("Input is lowered by Graph::run");
}

Variable::Variable(const Shape& shape, bool trainable)
    : Op("variable", shape), data_(tensor_alloc(shape.total())), trainable_(trainable)
{
}

Variable::~Variable()
{
    tensor_free(data_);
}

void Variable::compile()
{
    Graph::instance().add_compiled(this, {}, {}, nullptr, shape_get(), data_);
}

void Variable::write(const dbl_t* host) { tensor_write(data_begin(), data_end(), host); }
void Variable::read(dbl_t* host) const { tensor_read(data_, data_ + shape_get().total(), host); }

// ---- Graph -----------------------------------------------------------------------------------------
Graph& Graph::instance()
{
    static Graph g;
    return g;
}

Graph::~Graph()
{
    // The singleton dies during static destruction, possibly after the HIP runtime: device memory
    // is released by exit_graph() while the program runs, or by the driver at process exit.
}

void Graph::add(Op* op) { ops_.push_back(op); }
void Graph::add_var(Variable* var) { vars_.push_back(var); }

std::vector<Variable*> Graph::train_vars_get(Op* cost)
{
    std::vector<Variable*> res;
    for (Variable* v : vars_)
        if (v->is_trainable() && (!cost || v->pred_of(cost)))
            res.push_back(v);
    return res;
}

void Graph::add_compiled(Op* op, const std::vector<rt::Node*> nodes, std::vector<dbl_t*> tensors, rt::Node* out_node,
                         const Shape& out_shape, dbl_t* out_data)
{
    CompiledOp c;
    c.op = op;
    c.nodes = nodes;
    c.tensors = tensors;
    c.out_node = out_node;
    c.out_shape = out_shape;
    c.out_data = out_data;
    if (!compiled_ops_.emplace(op, c).second)
        throw std::logic_error("operator lowered twice");
    for (rt::Node* n : nodes)
        full_rt_graph_->add(n);
}

const CompiledOp& Graph::compiled(Op* op)
{
    auto it = compiled_ops_.find(op);
    if (it == compiled_ops_.end())
        throw std::logic_error("operator '" + op->name_get() + "' is not lowered yet");
    return it->second;
}

void Graph::compile_(Op* node)
{
    if (compiled_ops_.count(node))
        return;
    for (Op* p : node->preds())
        compile_(p);
    if (auto in = dynamic_cast<Input*>(node))
    {
        auto it = input_shapes_.find(in);
        if (it == input_shapes_.end())
            throw std::runtime_error("Graph::run: no data bound to an input the requested operators need");
        dbl_t* data = tensor_alloc(it->second.total());
        add_compiled(in, {}, {data}, nullptr, it->second, data);
        return;
    }
    node->compile();
}

void Graph::remove_compiled_rec_(Op* op)
{
    auto it = compiled_ops_.find(op);
    if (it == compiled_ops_.end())
        return;
    // the instructions of `op` and of everything downstream die with it
    for (rt::Node* n : it->second.nodes)
        full_rt_graph_->remove(n);
    for (dbl_t* t : it->second.tensors)
        tensor_free(t);
    compiled_ops_.erase(it);
    for (Op* s : op->succs())
        remove_compiled_rec_(s);
}

void Graph::run(std::vector<Op*> ops, const std::map<Input*, std::pair<const dbl_t*, Shape>>& inputs,
                const std::vector<dbl_t*>& outputs)
{
    // an input whose shape changed invalidates everything lowered from it
    bool relowered = false;
    for (const auto& kv : inputs)
    {
        auto old = input_shapes_.find(kv.first);
        if (old != input_shapes_.end() && old->second != kv.second.second && compiled_ops_.count(kv.first))
        {
            if (program_mode() == ProgramMode::GPU)
                hip::synchronize();
            remove_compiled_rec_(kv.first);
            relowered = true;
        }
        input_shapes_[kv.first] = kv.second.second;
    }
    if (relowered)
    {
        schedules_.clear();
        hip::forget_plans();
    }

    std::vector<rt::Node*> targets;
    for (Op* o : ops)
    {
        compile_(o);
        const CompiledOp& c = compiled(o);
        if (c.out_node)
            targets.push_back(c.out_node);
    }

    // From the first input noted to the end of the run the backend holds borrowed host pointers: an
    // exception on the way (an operator that cannot be lowered, a cycle, a failing launch) drops them.
    try
    {
        for (const auto& kv : inputs)
        {
            compile_(kv.first);
            dbl_t* dst = compiled(kv.first).out_data;
            // DCGAN_HIP_FEED=front: the copy in front of the run, as the reference places it
            static const bool deferred = !(std::getenv("DCGAN_HIP_FEED") && !std::strcmp(std::getenv("DCGAN_HIP_FEED"), "front"));
            if (program_mode() == ProgramMode::GPU && deferred)
                hip::feed(dst, kv.second.first, (std::size_t)kv.second.second.total());
            else
                tensor_write(dst, dst + kv.second.second.total(), kv.second.first);
        }

        // the execution order depends only on the requested operators: computed once, then reused
        auto sched = schedules_.find(ops);
        if (sched == schedules_.end())
            sched = schedules_.emplace(ops, full_rt_graph_->topological_sort(targets)).first;
        last_schedule_ = sched->second;
        rt::NodesList list(sched->second);
        if (debug_)
        {
            const ProgramMode m = program_mode();
            std::cout << "run program in "
                      << (m == ProgramMode::GPU ? "gpu" : m == ProgramMode::MULTITHREAD ? "multithread" : "monothread")
                      << "\n" << list;
        }

        std::vector<const dbl_t*> wanted;
        for (std::size_t i = 0; i < outputs.size() && i < ops.size(); ++i)
            if (outputs[i])
                wanted.push_back(compiled(ops[i]).out_data);
        if (name_results_)
            hip::set_protected_tensors(wanted);
        else
            hip::protect_all_tensors();
        if (!wanted.empty() && program_mode() == ProgramMode::GPU && hip::sync_each_run())
        {
            // the blocking device-to-host copy of the first result waits for the run: no separate wait
            hip::set_sync_each_run(false);
            try
            {
                rt::execute(list);
            }
            catch (...)
            {
                hip::set_sync_each_run(true);
                throw;
            }
            hip::set_sync_each_run(true);
        }
        else
            rt::execute(list);
    }
    catch (...)
    {
        hip::drop_feeds();
        throw;
    }

    for (std::size_t i = 0; i < outputs.size() && i < ops.size(); ++i)
    {
        if (!outputs[i])
            continue;
        const CompiledOp& c = compiled(ops[i]);
        tensor_read(c.out_data, c.out_data + c.out_shape.total(), outputs[i]);
    }
}

Op* Graph::gradient(Op* out, Op* var)
{
    auto key = std::make_pair(out, var);
    auto it = grads_.find(key);
    if (it != grads_.end())
        return it->second;
    Op* res = compute_gradient_(out, var);
    grads_[key] = res;
    return res;
}

Op* Graph::compute_gradient_(Op* out, Op* var)
{
    // Two paths from var to out: out is the sum of two costs (the real and the fake branch of the
    // discriminator), so the gradient is the sum of the two branch gradients
    // (src/ops/graph.cu:302-308 -- like the reference, only this two-operand case is handled).
    if (var->preds_of(out).size() > 1)
    {
        if (out->preds().size() != 2)
            throw std::runtime_error("Can't compute the gradient: several paths to a node that is not a sum");
        Op* left = gradient(out->preds()[0], var);
        Op* right = gradient(out->preds()[1], var);
        return OpsBuilder::instance().add(left, right);
    }
    std::size_t vari = out->pred_index(var);
    if (vari != std::size_t(-1))
        return out->child_grad(vari, nullptr);
    Op* succ = var->pred_of(out);
    if (!succ)
        throw std::runtime_error("Can't compute the gradient: the nodes are not related");
    Op* succ_grad = gradient(out, succ);
    vari = succ->pred_index(var);
    return succ->child_grad(vari, succ_grad);
}

namespace
{
bool is_npz(const std::string& path)
{
    return path.size() > 4 && path.compare(path.size() - 4, 4, ".npz") == 0;
}

npz::Array to_array(const std::string& name, Variable* v)
{
    npz::Array a;
    a.name = name;
    const Shape& sh = v->shape_get();
    for (std::size_t d = 0; d < sh.ndims(); ++d)
        a.shape.push_back((std::size_t)sh[d]);
    a.data.resize((std::size_t)sh.total());
    v->read(a.data.data());
    return a;
}

void from_array(const npz::Array& a, Variable* v, const std::string& path)
{
    if (a.data.size() != (std::size_t)v->shape_get().total())
        throw std::runtime_error("load: '" + a.name + "' in " + path + " has " + std::to_string(a.data.size()) +
                                 " values, the variable " + std::to_string(v->shape_get().total()));
    v->write(a.data.data());
}
}  // namespace

// `.npz` paths: one float32 array per trainable variable, in creation order, under numpy's positional
// names arr_0, arr_1, ... (the order-based convention of the reference's tensor files,
// src/ops/graph.cu:326-361).  Other paths: a `DGV1` header, then per variable the element count and
// the fp32 data.
void Graph::save_vars(const std::string& path)
{
    auto vars = train_vars_get(nullptr);
    if (is_npz(path))
    {
        std::vector<npz::Array> arrays;
        for (std::size_t i = 0; i < vars.size(); ++i)
            arrays.push_back(to_array("arr_" + std::to_string(i), vars[i]));
        npz::save(path, arrays);
        return;
    }
    std::FILE* f = std::fopen(path.c_str(), "wb");
    if (!f)
        throw std::runtime_error("save_vars: cannot open " + path);
    const std::uint64_t count = vars.size();
    std::fwrite("DGV1", 1, 4, f);
    std::fwrite(&count, sizeof(count), 1, f);
    for (Variable* v : vars)
    {
        const std::uint64_t n = v->shape_get().total();
        std::vector<dbl_t> host(n);
        v->read(host.data());
        std::fwrite(&n, sizeof(n), 1, f);
        std::fwrite(host.data(), sizeof(dbl_t), n, f);
    }
    std::fclose(f);
}

void Graph::load_vars(const std::string& path)
{
    auto vars = train_vars_get(nullptr);
    if (is_npz(path))
    {
        const std::vector<npz::Array> arrays = npz::load(path);
        if (arrays.size() != vars.size())
            throw std::runtime_error("load_vars: " + path + " holds " + std::to_string(arrays.size()) + " arrays, the graph " +
                                     std::to_string(vars.size()) + " trainable variables");
        for (std::size_t i = 0; i < vars.size(); ++i)
        {
            // by name when the archive uses the positional names, else by position
            const npz::Array* a = &arrays[i];
            for (const npz::Array& c : arrays)
                if (c.name == "arr_" + std::to_string(i))
                    a = &c;
            from_array(*a, vars[i], path);
        }
        return;
    }
    std::FILE* f = std::fopen(path.c_str(), "rb");
    if (!f)
        throw std::runtime_error("load_vars: cannot open " + path);
    std::unique_ptr<std::FILE, int (*)(std::FILE*)> guard(f, std::fclose);
    char magic[4];
    std::uint64_t count = 0;
    if (std::fread(magic, 1, 4, f) != 4 || std::string(magic, 4) != "DGV1" ||
        std::fread(&count, sizeof(count), 1, f) != 1 || count != vars.size())
        throw std::runtime_error("load_vars: " + path + " does not match this graph's variables");
    for (Variable* v : vars)
    {
        std::uint64_t n = 0;
        if (std::fread(&n, sizeof(n), 1, f) != 1 || n != (std::uint64_t)v->shape_get().total())
            throw std::runtime_error("load_vars: variable size mismatch in " + path);
        std::vector<dbl_t> host(n);
        if (std::fread(host.data(), sizeof(dbl_t), n, f) != n)
            throw std::runtime_error("load_vars: truncated file " + path);
        v->write(host.data());
    }
}

// Everything a training run needs to continue: all variables (the optimisers' moment estimates are
// non-trainable variables) as var_0, var_1, ... and the step counters of the Adam operators as
// adam_t.  The reference saves the trainable variables only, so its optimiser restarts from zero
// moments after a reload.
void Graph::save_state(const std::string& path)
{
    std::vector<npz::Array> arrays;
    for (std::size_t i = 0; i < vars_.size(); ++i)
        arrays.push_back(to_array("var_" + std::to_string(i), vars_[i]));
    npz::Array t;
    t.name = "adam_t";
    t.shape = {counters_.size()};
    for (const auto& c : counters_)
        t.data.push_back(*c);
    arrays.push_back(t);
    npz::save(path, arrays);
}

void Graph::load_state(const std::string& path)
{
    const std::vector<npz::Array> arrays = npz::load(path);
    auto find = [&](const std::string& name) -> const npz::Array& {
        for (const npz::Array& a : arrays)
            if (a.name == name)
                return a;
        throw std::runtime_error("load_state: no array '" + name + "' in " + path);
    };
    const npz::Array& t = find("adam_t");
    if (t.data.size() != counters_.size())
        throw std::runtime_error("load_state: " + path + " holds " + std::to_string(t.data.size()) +
                                 " step counters, the graph " + std::to_string(counters_.size()));
    for (std::size_t i = 0; i < vars_.size(); ++i)
        from_array(find("var_" + std::to_string(i)), vars_[i], path);
    if (program_mode() == ProgramMode::GPU && !compiled_ops_.empty())
        hip::synchronize();   // no run may be reading a counter while it changes
    for (std::size_t i = 0; i < counters_.size(); ++i)
        *counters_[i] = t.data[i];
}

void Graph::exit_graph()
{
    if (program_mode() == ProgramMode::GPU && !compiled_ops_.empty())
        hip::synchronize();
    for (auto& kv : compiled_ops_)
        for (dbl_t* t : kv.second.tensors)
            tensor_free(t);
    compiled_ops_.clear();
    delete full_rt_graph_;
    full_rt_graph_ = new rt::Graph;
    for (Op* o : ops_)
        delete o;
    ops_.clear();
    vars_.clear();
    counters_.clear();
    input_shapes_.clear();
    grads_.clear();
    schedules_.clear();
    last_schedule_.clear();
    hip::forget_plans();
}

// ---- OpsBuilder ------------------------------------------------------------------------------------
OpsBuilder& OpsBuilder::instance()
{
    static OpsBuilder b;
    return b;
}

namespace
{

Graph& G() { return Graph::instance(); }
OpsBuilder& B() { return OpsBuilder::instance(); }

void require(bool ok, const char* msg)
{
    if (!ok)
        throw std::runtime_error(msg);
}

Op* make(const std::string& name, const Shape& shape, const std::vector<Op*>& preds, Op::CompileFn c,
         Op::GradFn g = nullptr)
{
    Op* op = new Op(name, shape, preds);
    op->compile_fn = std::move(c);
    op->grad_fn = std::move(g);
    G().add(op);
    return op;
}

const CompiledOp& CP(Op& op, std::size_t i) { return G().compiled(op.preds()[i]); }

// Emit one instruction whose result is a freshly allocated tensor of `shape`.
template <class F>
void emit(Op& op, const Shape& shape, F node_for)
{
    dbl_t* out = tensor_alloc(shape.total() > 0 ? shape.total() : 1);
    rt::Node* n = node_for(out);
    G().add_compiled(&op, {n}, {out}, n, shape, out);
}

void dims4(const Shape& s, int out[4])
{
    for (int i = 0; i < 4; ++i)
        out[i] = s[i];
}

Op* need_dout(Op* dout, const char* msg)
{
    if (!dout)
        throw std::runtime_error(msg);
    return dout;
}

int ceil_div(int a, int b) { return (a + b - 1) / b; }

// TF "SAME" total padding of one axis (src/ops/conv2d.cu:33-41)
int same_pad_total(int in, int k, int s)
{
    return std::max(in % s == 0 ? k - s : k - in % s, 0);
}

Op* elementwise1(const char* name, Op* arg, rt::Node* (*factory)(const dbl_t*, dbl_t*, std::size_t, const rt::Node::Preds&),
                 Op::GradFn grad)
{
    return make(name, arg->shape_get(), {arg},
                [factory](Op& op) {
                    const CompiledOp& a = CP(op, 0);
                    emit(op, a.out_shape, [&](dbl_t* out) {
                        return factory(a.out_data, out, a.out_shape.total(), {a.out_node});
                    });
                },
                std::move(grad));
}

Op* elementwise2(const char* name, Op* a, Op* b,
                 rt::Node* (*factory)(const dbl_t*, const dbl_t*, dbl_t*, std::size_t, const rt::Node::Preds&),
                 Op::GradFn grad = nullptr)
{
    return make(name, a->shape_get(), {a, b},
                [factory](Op& op) {
                    const CompiledOp &x = CP(op, 0), &y = CP(op, 1);
                    emit(op, x.out_shape, [&](dbl_t* out) {
                        return factory(x.out_data, y.out_data, out, x.out_shape.total(), {x.out_node, y.out_node});
                    });
                },
                std::move(grad));
}

}  // namespace

Input* OpsBuilder::input(const Shape& shape)
{
    Input* in = new Input(shape);
    G().add(in);
    return in;
}

Variable* OpsBuilder::variable(const Shape& shape, bool trainable)
{
    require(shape.defined(), "shape not fully defined");
    Variable* v = new Variable(shape, trainable);
    G().add(v);
    G().add_var(v);
    return v;
}

Add* OpsBuilder::add(Op* left, Op* right)
{
    require(left->shape_get() == right->shape_get(), "add: left and right must have the same shape");
    return elementwise2("add", left, right, rt::Node::op_add, [](Op&, std::size_t, Op* dout) { return dout; });
}

Conv2D* OpsBuilder::conv2d(Op* input, Op* kernel, const int* strides)
{
    require(input->shape_get().ndims() == 4, "Conv2D:input must be a 4D tensor");
    require(kernel->shape_get().ndims() == 4, "Conv2D:kernel must be a 4D tensor");
    const Shape &xs = input->shape_get(), &ks = kernel->shape_get();
    const std::vector<int> s = {strides[0], strides[1]};
    const std::vector<int> pads = {same_pad_total(xs[1], ks[0], s[0]), same_pad_total(xs[2], ks[1], s[1])};
    const Shape out({xs[0], ceil_div(xs[1], s[0]), ceil_div(xs[2], s[1]), ks[3]});
    return make(
        "conv2d", out, {input, kernel},
        [s, pads](Op& op) {
            const CompiledOp &x = CP(op, 0), &k = CP(op, 1);
            int xsz[4], ksz[4];
            dims4(x.out_shape, xsz);
            dims4(k.out_shape, ksz);
            const Shape o({xsz[0], ceil_div(xsz[1], s[0]), ceil_div(xsz[2], s[1]), ksz[3]});
            emit(op, o, [&](dbl_t* y) {
                return rt::Node::op_conv2d(x.out_data, k.out_data, s.data(), pads[0], pads[1], y, xsz, ksz,
                                           {x.out_node, k.out_node});
            });
        },
        [s, pads](Op& op, std::size_t index, Op* dout) -> Op* {
            need_dout(dout, "conv2d must not be the final node of the gradient");
            int xsz[4], ksz[4];
            dims4(op.preds()[0]->shape_get(), xsz);
            dims4(op.preds()[1]->shape_get(), ksz);
            if (index == 0)
                return B().conv2d_input_grad(dout, op.preds()[1], s.data(), xsz);
            return B().conv2d_kernel_grad(dout, op.preds()[0], s.data(), ksz, pads.data());
        });
}

Conv2DInputGrad* OpsBuilder::conv2d_input_grad(Op* y, Op* kernel, const int* strides, const int* input_size)
{
    const std::vector<int> s = {strides[0], strides[1]};
    const std::vector<int> in(input_size, input_size + 4);
    return make("conv2d_input_grad", Shape(in), {y, kernel}, [s, in](Op& op) {
        const CompiledOp &dy = CP(op, 0), &k = CP(op, 1);
        int ysz[4], ksz[4];
        dims4(dy.out_shape, ysz);
        dims4(k.out_shape, ksz);
        emit(op, Shape(in), [&](dbl_t* dx) {
            return rt::Node::op_conv2d_input_grad(dy.out_data, k.out_data, s.data(), dx, ysz, ksz, in.data(),
                                                  {dy.out_node, k.out_node});
        });
    });
}

Conv2DKernelGrad* OpsBuilder::conv2d_kernel_grad(Op* y, Op* input, const int* strides, const int* kernel_size,
                                                 const int* padded_size)
{
    const std::vector<int> s = {strides[0], strides[1]};
    const std::vector<int> ks(kernel_size, kernel_size + 4);
    const std::vector<int> pads = {padded_size[0], padded_size[1]};
    return make("conv2d_kernel_grad", Shape(ks), {y, input}, [s, ks, pads](Op& op) {
        const CompiledOp &dy = CP(op, 0), &x = CP(op, 1);
        int ysz[4], xsz[4];
        dims4(dy.out_shape, ysz);
        dims4(x.out_shape, xsz);
        emit(op, Shape(ks), [&](dbl_t* dk) {
            return rt::Node::op_conv2d_kernel_grad(dy.out_data, x.out_data, s.data(), dk, ysz, xsz, pads.data(),
                                                   {dy.out_node, x.out_node});
        });
    });
}

Conv2DTranspose* OpsBuilder::conv2d_transpose(Op* input, Op* kernel, const int* out_size, const int* strides)
{
    const std::vector<int> s = {strides[0], strides[1]};
    const std::vector<int> os(out_size, out_size + 4);
    return make(
        "conv2d_transpose", Shape(os), {input, kernel},
        [s, os](Op& op) {
            const CompiledOp &x = CP(op, 0), &k = CP(op, 1);
            int xsz[4], ksz[4];
            dims4(x.out_shape, xsz);
            dims4(k.out_shape, ksz);
            emit(op, Shape(os), [&](dbl_t* y) {
                return rt::Node::op_conv2d_transpose(x.out_data, k.out_data, os.data(), s.data(), y, xsz, ksz,
                                                     {x.out_node, k.out_node});
            });
        },
        [s](Op& op, std::size_t index, Op* dout) -> Op* {
            need_dout(dout, "conv2d_transpose must not be the final node of the gradient");
            int xsz[4], ksz[4];
            dims4(op.preds()[0]->shape_get(), xsz);
            dims4(op.preds()[1]->shape_get(), ksz);
            if (index == 0)
                return B().conv2d_transpose_input_grad(dout, op.preds()[1], s.data(), xsz);
            return B().conv2d_transpose_kernel_grad(dout, op.preds()[0], s.data(), ksz);
        });
}

Conv2DTransposeInputGrad* OpsBuilder::conv2d_transpose_input_grad(Op* y, Op* kernel, const int* strides,
                                                                  const int* input_size)
{
    const std::vector<int> s = {strides[0], strides[1]};
    const std::vector<int> in(input_size, input_size + 4);
    return make("conv2d_transpose_input_grad", Shape(in), {y, kernel}, [s, in](Op& op) {
        const CompiledOp &dy = CP(op, 0), &k = CP(op, 1);
        int ysz[4], ksz[4];
        dims4(dy.out_shape, ysz);
        dims4(k.out_shape, ksz);
        emit(op, Shape(in), [&](dbl_t* dx) {
            return rt::Node::op_conv2d_transpose_input_grad(dy.out_data, k.out_data, s.data(), dx, ysz, ksz,
                                                            in.data(), {dy.out_node, k.out_node});
        });
    });
}

Conv2DTransposeKernelGrad* OpsBuilder::conv2d_transpose_kernel_grad(Op* y, Op* input, const int* strides,
                                                                    const int* kernel_size)
{
    const std::vector<int> s = {strides[0], strides[1]};
    const std::vector<int> ks(kernel_size, kernel_size + 4);
    return make("conv2d_transpose_kernel_grad", Shape(ks), {y, input}, [s, ks](Op& op) {
        const CompiledOp &dy = CP(op, 0), &x = CP(op, 1);
        int ysz[4], xsz[4];
        dims4(dy.out_shape, ysz);
        dims4(x.out_shape, xsz);
        emit(op, Shape(ks), [&](dbl_t* dk) {
            return rt::Node::op_conv2d_transpose_kernel_grad(dy.out_data, x.out_data, s.data(), dk, ysz, xsz,
                                                             ks.data(), {dy.out_node, x.out_node});
        });
    });
}

// Lowered to mat_rvect_add over [N*H*W, C] (src/ops/conv2d-bias-add.cu:35-38)
Conv2DBiasAdd* OpsBuilder::conv2d_bias_add(Op* z, Op* bias)
{
    require(z->shape_get().ndims() == 4, "Conv2DBiasAdd:z must be a 4D tensor");
    require(bias->shape_get().ndims() == 1, "Conv2DBiasAdd:bias must be a 1D array");
    require(z->shape_get()[3] == bias->shape_get()[0], "Conv2DBiasAdd:z and bias shape are not corresponding");
    return make(
        "conv2d_bias_add", z->shape_get(), {z, bias},
        [](Op& op) {
            const CompiledOp &cz = CP(op, 0), &cb = CP(op, 1);
            const Shape& s = cz.out_shape;
            emit(op, s, [&](dbl_t* out) {
                return rt::Node::op_mat_rvect_add(cz.out_data, cb.out_data, out, (std::size_t)s[0] * s[1] * s[2], s[3],
                                                  {cz.out_node, cb.out_node});
            });
        },
        [](Op&, std::size_t index, Op* dout) -> Op* {
            need_dout(dout, "conv2d_bias_add must not be the final node of the gradient");
            return index == 0 ? dout : B().conv2d_bias_add_grad(dout);
        });
}

// Lowered to mat_sum_cols over [N*H*W, C] (src/ops/conv2d-bias-add-grad.cu:29-31)
Conv2DBiasAddGrad* OpsBuilder::conv2d_bias_add_grad(Op* z)
{
    require(z->shape_get().ndims() == 4, "Conv2DBiasAddGrad:z must be a 4D tensor");
    return make("conv2d_bias_add_grad", Shape({z->shape_get()[3]}), {z}, [](Op& op) {
        const CompiledOp& cz = CP(op, 0);
        const Shape& s = cz.out_shape;
        emit(op, Shape({s[3]}), [&](dbl_t* out) {
            return rt::Node::op_mat_sum_cols(cz.out_data, out, (std::size_t)s[0] * s[1] * s[2], s[3], {cz.out_node});
        });
    });
}

MatMatMul* OpsBuilder::mat_mat_mul(Op* left, Op* right, bool left_tr, bool right_tr)
{
    require(left->shape_get().ndims() == 2, "left operand must be a matrix");
    require(right->shape_get().ndims() == 2, "right operand must be a matrix");
    require(left->shape_get()[!left_tr] == right->shape_get()[right_tr], "left[1] and right[0] differ");
    require(!(left_tr && right_tr), "mat_mat_mul: transposing both operands is not supported");
    const Shape out({left->shape_get()[left_tr], right->shape_get()[!right_tr]});
    return make(
        "mat_mat_mul", out, {left, right},
        [left_tr, right_tr](Op& op) {
            const CompiledOp &l = CP(op, 0), &r = CP(op, 1);
            const std::size_t n = l.out_shape[left_tr], p = l.out_shape[!left_tr], q = r.out_shape[!right_tr];
            auto factory = left_tr ? rt::Node::op_tmat_mat_mul : right_tr ? rt::Node::op_mat_tmat_mul
                                                                          : rt::Node::op_mat_mat_mul;
            emit(op, Shape({int(n), int(q)}), [&](dbl_t* out_data) {
                return factory(l.out_data, r.out_data, out_data, n, p, q, {l.out_node, r.out_node});
            });
        },
        [left_tr, right_tr](Op& op, std::size_t index, Op* dout) -> Op* {
            need_dout(dout, "MatMatMul can't be the final node of the gradient");
            require(!left_tr && !right_tr, "gradient of a transposed product is not supported");
            if (index == 0)
                return B().mat_mat_mul(dout, op.preds()[1], false, true);
            return B().mat_mat_mul(op.preds()[0], dout, true, false);
        });
}

MatMulAdd* OpsBuilder::mat_mul_add(Op* x, Op* w, Op* b)
{
    require(x->shape_get().ndims() == 2, "x must be a matrix");
    require(w->shape_get().ndims() == 2, "w must be a matrix");
    require(b->shape_get().ndims() == 1, "b must be a vector");
    require(x->shape_get()[1] == w->shape_get()[0], "x[1] and w[0] differ");
    require(w->shape_get()[1] == b->shape_get()[0], "w[1] and b[0] differ");
    return make(
        "mat_mul_add", Shape({x->shape_get()[0], w->shape_get()[1]}), {x, w, b},
        [](Op& op) {
            const CompiledOp &cx = CP(op, 0), &cw = CP(op, 1), &cb = CP(op, 2);
            const std::size_t m = cx.out_shape[0], n = cx.out_shape[1], p = cw.out_shape[1];
            emit(op, Shape({int(m), int(p)}), [&](dbl_t* out) {
                return rt::Node::op_mat_mul_add(cx.out_data, cw.out_data, cb.out_data, out, m, n, p,
                                                {cx.out_node, cw.out_node, cb.out_node});
            });
        },
        [](Op& op, std::size_t index, Op* dout) -> Op* {
            need_dout(dout, "MatMullAdd can't be the final node of the gradient");
            if (index == 0)
                return B().mat_mat_mul(dout, op.preds()[1], false, true);
            if (index == 1)
                return B().mat_mat_mul(op.preds()[0], dout, true, false);
            return B().mat_sum(dout, 0);
        });
}

MatRvectAdd* OpsBuilder::mat_rvect_add(Op* left, Op* right)
{
    require(left->shape_get().ndims() == 2, "left operand must be a matrix");
    require(right->shape_get().ndims() == 1, "right operand must be a vector");
    require(left->shape_get()[1] == right->shape_get()[0], "left[1] and right[0] differ");
    return make(
        "mat_rvect_add", left->shape_get(), {left, right},
        [](Op& op) {
            const CompiledOp &l = CP(op, 0), &r = CP(op, 1);
            emit(op, l.out_shape, [&](dbl_t* out) {
                return rt::Node::op_mat_rvect_add(l.out_data, r.out_data, out, l.out_shape[0], l.out_shape[1],
                                                  {l.out_node, r.out_node});
            });
        },
        [](Op&, std::size_t index, Op* dout) -> Op* {
            need_dout(dout, "MatRvectAdd can't be the final node of the gradient");
            return index == 0 ? dout : B().mat_sum(dout, 0);
        });
}

MatSum* OpsBuilder::mat_sum(Op* arg, std::size_t axis)
{
    require(arg->shape_get().ndims() == 2, "arg must be a matrix");
    require(axis < 2, "axis must be 0 or 1");
    return make("mat_sum", Shape({arg->shape_get()[!axis]}), {arg}, [axis](Op& op) {
        const CompiledOp& a = CP(op, 0);
        const std::size_t rows = a.out_shape[0], cols = a.out_shape[1];
        emit(op, Shape({a.out_shape[!axis]}), [&](dbl_t* out) {
            return axis == 0 ? rt::Node::op_mat_sum_cols(a.out_data, out, rows, cols, {a.out_node})
                             : rt::Node::op_mat_sum_rows(a.out_data, out, rows, cols, {a.out_node});
        });
    });
}

VectRelu* OpsBuilder::vect_relu(Op* arg)
{
    return elementwise1("vect_relu", arg, rt::Node::op_relu, [](Op& op, std::size_t, Op* dout) -> Op* {
        need_dout(dout, "grad(Relu) can't be computed on last node");
        return B().relu_grad(op.preds()[0], dout);
    });
}

VectReluLeaky* OpsBuilder::vect_relu_leaky(Op* arg, const dbl_t alpha)
{
    return make(
        "vect_relu_leaky", arg->shape_get(), {arg},
        [alpha](Op& op) {
            const CompiledOp& a = CP(op, 0);
            emit(op, a.out_shape, [&](dbl_t* out) {
                return rt::Node::op_relu_leaky(a.out_data, out, a.out_shape.total(), alpha, {a.out_node});
            });
        },
        [alpha](Op& op, std::size_t, Op* dout) -> Op* {
            need_dout(dout, "grad(LeakyRelu) can't be computed on last node");
            return B().leaky_relu_grad(op.preds()[0], dout, alpha);
        });
}

VectTanh* OpsBuilder::vect_tanh(Op* arg)
{
    return elementwise1("vect_tanh", arg, rt::Node::op_tanh, [](Op& op, std::size_t, Op* dout) -> Op* {
        need_dout(dout, "grad(Tanh) can't be computed on last node");
        return B().tanh_grad(&op, dout);  // from the OUTPUT of tanh
    });
}

VectSigmoid* OpsBuilder::vect_sigmoid(Op* arg)
{
    return elementwise1("vect_sigmoid", arg, rt::Node::op_sigmoid, [](Op& op, std::size_t, Op* dout) -> Op* {
        need_dout(dout, "grad(Sigmoid) can't be computed on last node");
        return B().sigmoid_grad(&op, dout);  // from the OUTPUT of sigmoid
    });
}

ReluGrad* OpsBuilder::relu_grad(Op* z, Op* dout)
{
    require(z->shape_get() == dout->shape_get(), "ReluGrad: z and dout must have the same shape");
    return elementwise2("relu_grad", z, dout, rt::Node::op_relu_grad);
}

LeakyReluGrad* OpsBuilder::leaky_relu_grad(Op* z, Op* dout, dbl_t alpha)
{
    require(z->shape_get() == dout->shape_get(), "LeakyReluGrad: z and dout must have the same shape");
    return make("leaky_relu_grad", z->shape_get(), {z, dout}, [alpha](Op& op) {
        const CompiledOp &cz = CP(op, 0), &cd = CP(op, 1);
        emit(op, cz.out_shape, [&](dbl_t* out) {
            return rt::Node::op_leaky_relu_grad(cz.out_data, cd.out_data, out, alpha, cz.out_shape.total(),
                                                {cz.out_node, cd.out_node});
        });
    });
}

TanhGrad* OpsBuilder::tanh_grad(Op* tanh_out, Op* dout)
{
    require(tanh_out->shape_get() == dout->shape_get(), "TanhGrad: tanh_out and dout must have the same shape");
    return elementwise2("tanh_grad", tanh_out, dout, rt::Node::op_tanh_grad);
}

SigmoidGrad* OpsBuilder::sigmoid_grad(Op* sig_out, Op* dout)
{
    require(sig_out->shape_get() == dout->shape_get(), "SigmoidGrad: sig_out and dout must have the same shape");
    return elementwise2("sigmoid_grad", sig_out, dout, rt::Node::op_sigmoid_grad);
}

SigmoidCrossEntropy* OpsBuilder::sigmoid_cross_entropy(Op* y, Op* logits)
{
    require(y->shape_get().ndims() == 2, "y must be a matrix");
    require(logits->shape_get().ndims() == 2, "logits must be a matrix");
    require(y->shape_get() == logits->shape_get(), "y and logits must have the same shape");
    return make(
        "sigmoid_cross_entropy", Shape(), {y, logits},
        [](Op& op) {
            const CompiledOp &cy = CP(op, 0), &cl = CP(op, 1);
            emit(op, Shape(), [&](dbl_t* out) {
                return rt::Node::op_sigmoid_cross_entropy(cy.out_data, cl.out_data, out, cy.out_shape.total(),
                                                          {cy.out_node, cl.out_node});
            });
        },
        [](Op& op, std::size_t index, Op* dout) -> Op* {
            require(index != 0, "Can't compute gradient of sigmoid_cross_entropy for y");
            require(dout == nullptr, "sigmoid_cross_entropy must be the final node of the gradient");
            return B().sigmoid_cross_entropy_grad(op.preds()[0], op.preds()[1]);
        });
}

SigmoidCrossEntropyGrad* OpsBuilder::sigmoid_cross_entropy_grad(Op* y, Op* logits)
{
    require(y->shape_get().ndims() == 2, "y must be a matrix");
    require(logits->shape_get().ndims() == 2, "logits must be a matrix");
    require(y->shape_get() == logits->shape_get(), "y and logits must have the same shape");
    return elementwise2("sigmoid_cross_entropy_grad", y, logits, rt::Node::op_sigmoid_cross_entropy_grad);
}

MSE* OpsBuilder::mse(Op* y, Op* y_hat)
{
    require(y->shape_get().ndims() == 2, "MSE:y must be a matrix");
    require(y_hat->shape_get().ndims() == 2, "MSE:y_hat must be a matrix");
    require(y->shape_get() == y_hat->shape_get(), "MSE: y and y_hat must have the same shape");
    return make(
        "mse", Shape(), {y, y_hat},
        [](Op& op) {
            const CompiledOp &cy = CP(op, 0), &ch = CP(op, 1);
            emit(op, Shape(), [&](dbl_t* out) {
                return rt::Node::op_mse(cy.out_data, ch.out_data, out, cy.out_shape[0], cy.out_shape[1],
                                        {cy.out_node, ch.out_node});
            });
        },
        [](Op& op, std::size_t index, Op* dout) -> Op* {
            require(index != 0, "Can't compute gradient of MSE for y");
            require(dout == nullptr, "MSE must be the final node of the gradient");
            return B().mse_grad(op.preds()[0], op.preds()[1]);
        });
}

MSEGrad* OpsBuilder::mse_grad(Op* y, Op* y_hat)
{
    require(y->shape_get().ndims() == 2, "MSEGrad: y must be a matrix");
    require(y_hat->shape_get().ndims() == 2, "MSEGrad: y_hat must be a matrix");
    require(y->shape_get() == y_hat->shape_get(), "MSEGrad: y and y_hat must have the same shape");
    return elementwise2("mse_grad", y, y_hat, rt::Node::op_mse_grad);
}

ArgmaxAccuracy* OpsBuilder::argmax_accuracy(Op* y, Op* y_hat)
{
    require(y->shape_get().ndims() == 2, "y must be a matrix");
    require(y_hat->shape_get().ndims() == 2, "y_hat must be a matrix");
    require(y->shape_get() == y_hat->shape_get(), "y and y_hat must have the same shape");
    return make("argmax_accuracy", Shape(), {y, y_hat}, [](Op& op) {
        const CompiledOp &cy = CP(op, 0), &ch = CP(op, 1);
        emit(op, Shape(), [&](dbl_t* out) {
            return rt::Node::op_argmax_acc(cy.out_data, ch.out_data, out, cy.out_shape[0], cy.out_shape[1],
                                           {cy.out_node, ch.out_node});
        });
    });
}

// A view: no instruction, the result aliases the operand (src/ops/reshape.cu:20-44)
Reshape* OpsBuilder::reshape(Op* arg, const Shape& shape)
{
    if (shape.defined() && shape.total() != arg->shape_get().total())
        throw std::runtime_error("Reshape:");
    const Shape initial = arg->shape_get();
    return make(
        "reshape", shape, {arg},
        [shape](Op& op) {
            const CompiledOp& a = CP(op, 0);
            std::vector<int> dims = shape.dims();
            if (!shape.defined())
                for (int& d : dims)
                    if (d == -1)
                        d = a.out_shape.total() / (-shape.total());
            rt::Node* n = rt::Node::nop({a.out_node});
            G().add_compiled(&op, {n}, {}, n, Shape(dims), a.out_data);
        },
        [initial](Op&, std::size_t, Op* dout) -> Op* {
            need_dout(dout, "reshape dout must not be null");
            return B().reshape(dout, initial);
        });
}

// Runs all operands; the value is the last one's (src/ops/seq.cu:17-28)
Seq* OpsBuilder::seq(const std::vector<Op*>& ops)
{
    require(!ops.empty(), "seq: ops can't be empty");
    return make("seq", ops.back()->shape_get(), ops, [](Op& op) {
        std::vector<rt::Node*> nodes;
        for (Op* p : op.preds())
            nodes.push_back(G().compiled(p).out_node);
        const CompiledOp& last = G().compiled(op.preds().back());
        rt::Node* n = rt::Node::nop(nodes);
        G().add_compiled(&op, {n}, {}, n, last.out_shape, last.out_data);
    });
}

// In-place on the variable's storage (src/ops/moment-update.cu:23-44)
MomentUpdate* OpsBuilder::moment_update(Variable* var, Op* dt, dbl_t coeff1, dbl_t coeff2, bool sq_update)
{
    require(var->shape_get() == dt->shape_get(), "var and dt must have the same shape");
    return make("moment_update", var->shape_get(), {var, dt}, [var, coeff1, coeff2, sq_update](Op& op) {
        const CompiledOp& g = CP(op, 1);
        const std::size_t len = g.out_shape.total();
        dbl_t* ptr = var->data_begin();
        rt::Node* n = sq_update ? rt::Node::op_moment_update2(ptr, g.out_data, coeff1, coeff2, len, {g.out_node})
                                : rt::Node::op_moment_update(ptr, g.out_data, coeff1, coeff2, len, {g.out_node});
        G().add_compiled(&op, {n}, {}, n, g.out_shape, ptr);
    });
}

// The step counter t is host state owned by the operator (src/ops/adam-update.cu:14-50)
AdamUpdate* OpsBuilder::adam_update(Variable* var, Op* m, Op* v, dbl_t learning_rate, dbl_t beta1, dbl_t beta2,
                                    dbl_t eps)
{
    require(var->shape_get() == m->shape_get(), "var and m must have the same shape");
    require(var->shape_get() == v->shape_get(), "var and v must have the same shape");
    auto t = std::make_shared<dbl_t>(0);
    G().add_counter(t);
    return make("adam_update", var->shape_get(), {var, m, v}, [var, t, learning_rate, beta1, beta2, eps](Op& op) {
        const CompiledOp &cm = CP(op, 1), &cv = CP(op, 2);
        dbl_t* ptr = var->data_begin();
        rt::Node* n = rt::Node::op_adam_update(ptr, t.get(), cm.out_data, cv.out_data, learning_rate, beta1, beta2,
                                               eps, cm.out_shape.total(), {cm.out_node, cv.out_node});
        G().add_compiled(&op, {n}, {}, n, cm.out_shape, ptr);
    });
}

// SGD step with a device-resident scalar coefficient (src/ops/update.cu)
Update* OpsBuilder::update(Variable* var, Op* dt, Op* coeff)
{
    require(var->shape_get() == dt->shape_get(), "var and dt must have the same shape");
    require(coeff->shape_get().ndims() == 0, "coeff must be a scalar");
    return make("update", var->shape_get(), {var, dt, coeff}, [var](Op& op) {
        const CompiledOp &g = CP(op, 1), &c = CP(op, 2);
        dbl_t* ptr = var->data_begin();
        rt::Node* n = rt::Node::op_update(ptr, g.out_data, c.out_data, g.out_shape.total(), {g.out_node, c.out_node});
        G().add_compiled(&op, {n}, {}, n, g.out_shape, ptr);
    });
}

}  // namespace ops
