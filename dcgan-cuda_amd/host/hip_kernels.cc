// The HIP backend's planning runner: the instruction list of a run is pattern-matched into fused and
// paired C-ABI calls (or issued node by node through the kernel table of hip_table.cc when fusion is
// off), without the reference's per-node device synchronisation (src/gpu/runner.cu:10-18).
//
// Depends on rt::Node, rt::NodesList and the C ABI only (see hip_runner.hh): it compiles unchanged
// against the reference's src/runtime headers.
#include "hip_runner.hh"

#include <algorithm>
#include <array>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <unordered_set>

#include "dcgan_hip.h"

namespace hip
{

namespace
{

int g_fusion = -1;         // -1: not decided yet (reads DCGAN_HIP_FUSE)
int g_last_launches = 0;    // steps of the plan that ran last and launched something
bool g_pairing = true;     // issue same-filter convolutions of independent towers as one launch (part of fusion)

#define CK(call) check((call), #call)

// conv_fwd / conv_dx: one C-ABI call for a decoded geometry (with optional epilogue)
void conv_fwd(const ConvGeom& g, const dbl_t* x, const dbl_t* k, dbl_t* y, const dbl_t* bias, int act, float alpha)
{
    CK(dh_conv2d_fwd(x, k, y, g.N, g.H, g.W, g.C, g.kh, g.kw, g.O, g.sh, g.sw, g.pt, g.pl, g.Ho, g.Wo, bias, act,
                     alpha, g_stream));
}

void conv_dx(const ConvGeom& g, const dbl_t* dy, const dbl_t* k, dbl_t* dx, const dbl_t* bias, int act, float alpha)
{
    CK(dh_conv2d_dx(dy, k, dx, g.N, g.Ho, g.Wo, g.O, g.kh, g.kw, g.C, g.sh, g.sw, g.pt, g.pl, g.H, g.W, bias, act,
                    alpha, g_stream));
}



// ---- fusion plan -------------------------------------------------------------------------------
// A step is either one node run through the table or one fused call standing for several nodes.
struct Step
{
    enum Kind { NODE, CONV_EPILOGUE, ACT_BIAS_GRAD, ADAM, ADAM_MULTI, CONV_PAIR, DENSE_EPILOGUE, SCE_HEAD } kind = NODE;
    // NODE: the node; CONV_EPILOGUE: the conv node; ACT_BIAS_GRAD: the act-grad node; DENSE_EPILOGUE: the
    // mat_mul_add node (act: its activation); SCE_HEAD: the sigmoid_cross_entropy_grad node
    rt::Node* node = nullptr;
    rt::Node* bias = nullptr;    // CONV_EPILOGUE: the mat_rvect_add node (may be null)
    rt::Node* act = nullptr;     // CONV_EPILOGUE: the activation node (may be null)
    rt::Node* sum = nullptr;     // ACT_BIAS_GRAD: the mat_sum_cols node
    rt::Node* m1 = nullptr;      // ADAM: moment_update, moment_update2; node = adam_update
    rt::Node* m2 = nullptr;
    rt::Node* add = nullptr;     // ADAM: the `add` node that formed the gradient from two contributions (may be null)
                                 // SCE_HEAD of two towers: the `add` node that joins their losses
    rt::Node* loss = nullptr;    // SCE_HEAD: the sigmoid_cross_entropy node on the same labels and logits as `node`
    rt::Node* node2 = nullptr;   // SCE_HEAD of two towers: gradient and loss node of the second
    rt::Node* loss2 = nullptr;
    const dbl_t* act_ref = nullptr;  // ACT_BIAS_GRAD: tensor the activation gradient reads
    std::vector<Step> group;     // ADAM_MULTI: the ADAM steps issued as one launch; CONV_PAIR: the two convolution steps
    const dbl_t* grad_sum = nullptr;  // ADAM: gradient tensor that already holds the sum of both contributions
    // A bias gradient read by nothing but the optimiser is left as its row-range sums and added up
    // inside the optimiser launch (defer_bias_sums).  Producer (ACT_BIAS_GRAD, or NODE mat_sum_cols):
    // where the sums go.  ADAM: for each of its two gradient slots, the sums and their count.
    dbl_t* parts = nullptr;
    bool rows_as_parts = false;   // NODE mat_sum_cols of a matrix of few rows: no launch, the optimiser adds the rows up
    const dbl_t* g_parts[2] = {nullptr, nullptr};
    std::size_t g_nparts[2] = {0, 0};
};

int act_code(const rt::Node* n)
{
    switch (n->type)
    {
    case rt::Node::OP_RELU: return DH_ACT_RELU;
    case rt::Node::OP_RELU_LEAKY: return DH_ACT_LEAKY;
    case rt::Node::OP_TANH: return DH_ACT_TANH;
    case rt::Node::OP_SIGMOID: return DH_ACT_SIGMOID;
    default: return -1;
    }
}

bool is_conv_like(const rt::Node* n)
{
    return n->type == rt::Node::OP_CONV2D || n->type == rt::Node::OP_CONV2D_TRANSPOSE ||
           n->type == rt::Node::OP_CONV2D_TRANSPOSE_INPUT_GRAD || n->type == rt::Node::OP_CONV2D_INPUT_GRAD;
}

struct Plan
{
    std::vector<Step> steps;
};

// The tensors the caller may read once the run is over.  gpu::run receives nothing but the instruction
// list (src/gpu/runner.cu:10, src/ops/graph.cu:194-215 reads the results afterwards), so until the
// caller has named them with set_protected_tensors EVERY tensor counts: the plan then holds only the
// fusions that still write all outputs of the nodes they stand for.
struct Keep
{
    bool all = true;
    std::unordered_set<const dbl_t*> set;
    std::size_t count(const dbl_t* t) const { return all || set.count(t) ? 1 : 0; }
};

// Which instructions of the list read tensor `t`.
struct Readers
{
    std::unordered_map<const dbl_t*, std::vector<rt::Node*>> by_tensor;
    explicit Readers(const std::vector<rt::Node*>& nodes)
    {
        for (rt::Node* n : nodes)
            for (const dbl_t* t : {n->in1, n->in2, n->in3})
                if (t)
                    by_tensor[t].push_back(n);
    }
    const std::vector<rt::Node*>& of(const dbl_t* t) const
    {
        static const std::vector<rt::Node*> none;
        auto it = by_tensor.find(t);
        return it == by_tensor.end() ? none : it->second;
    }
};

// The nodes a step stands for (null where it has none in that role).
std::array<rt::Node*, 10> nodes_of(const Step& s)
{
    return {s.node, s.bias, s.act, s.sum, s.m1, s.m2, s.add, s.loss, s.node2, s.loss2};
}

// Every tensor a step reads or writes.
void tensors_of(const Step& s, std::unordered_set<const dbl_t*>& out)
{
    for (const rt::Node* n : nodes_of(s))
        if (n)
            for (const dbl_t* t : {(const dbl_t*)n->in1, (const dbl_t*)n->in2, (const dbl_t*)n->in3, (const dbl_t*)n->out1})
                if (t)
                    out.insert(t);
    if (s.act_ref)
        out.insert(s.act_ref);
}

// Moves the optimiser steps of a plan to its end and issues them as ONE launch.  A step stays where
// it is when anything after it touches its variable, its moments or its gradient: executing the list
// in order must give the same values as before.
void gather_adam_steps(Plan& plan)
{
    std::unordered_set<const dbl_t*> later;   // tensors touched by the steps that follow and stay
    std::vector<Step> kept, moved;
    for (auto it = plan.steps.rbegin(); it != plan.steps.rend(); ++it)
    {
        bool movable = it->kind == Step::ADAM;
        if (movable)
        {
            std::unordered_set<const dbl_t*> mine;
            tensors_of(*it, mine);
            for (const dbl_t* t : mine)
                if (later.count(t))
                    movable = false;
            // two optimiser steps on the same variable keep their order: leave both in place
            for (const Step& m : moved)
                if (m.node->out1 == it->node->out1)
                    movable = false;
        }
        if (movable)
            moved.push_back(*it);
        else
        {
            tensors_of(*it, later);
            kept.push_back(*it);
        }
    }
    if (moved.size() < 2)
        return;
    std::reverse(kept.begin(), kept.end());
    std::reverse(moved.begin(), moved.end());
    // one launch per set of hyper-parameters (all variables of an optimiser share them)
    while (!moved.empty())
    {
        Step multi;
        multi.kind = Step::ADAM_MULTI;
        multi.node = moved.front().node;
        std::vector<Step> rest;
        for (const Step& m : moved)
        {
            const Step& f = moved.front();
            const bool same = m.m1->cons1 == f.m1->cons1 && m.m1->cons2 == f.m1->cons2 && m.m2->cons1 == f.m2->cons1 &&
                              m.m2->cons2 == f.m2->cons2 && m.node->cons4 == f.node->cons4;
            (same ? multi.group : rest).push_back(m);
        }
        kept.push_back(multi);
        moved.swap(rest);
    }
    plan.steps.swap(kept);
}

// ---- bias gradients summed inside the optimiser launch ---------------------------------------------
// A bias gradient is a column sum in two kernels: sums over ranges of rows, then the sum of those.
// When nothing but optimiser steps of one launch reads it, the second kernel is dropped: the producer
// writes its row-range sums to a buffer of its own and dh_adam_step_multi adds them, in the same
// order, while it reads the gradient (15 launches of a DCGAN iteration, each of them pure latency).
std::unordered_map<const dbl_t*, std::pair<dbl_t*, std::size_t>> g_parts_pool;   // bias gradient -> (buffer, floats)

dbl_t* parts_buffer(const dbl_t* grad, std::size_t floats)
{
    auto& slot = g_parts_pool[grad];
    if (slot.second < floats)
    {
        if (slot.first)
            CK(dh_pool_free(slot.first));
        void* q = nullptr;
        CK(dh_pool_alloc(&q, floats * sizeof(dbl_t)));
        slot = {static_cast<dbl_t*>(q), floats};
    }
    return slot.first;
}

// Whether exactly one node of the plan writes the tensor.
bool written_once(const Plan& plan, const dbl_t* t)
{
    int writers = 0;
    auto count = [&](const Step& s) {
        for (const rt::Node* n : nodes_of(s))
            if (n && (n->out1 == t || n->out2 == t))
                writers += 1;
    };
    for (const Step& s : plan.steps)
    {
        count(s);
        for (const Step& g : s.group)
            count(g);
    }
    return writers == 1;
}

void defer_bias_sums(Plan& plan, const Keep& keep)
{
    // the optimiser steps of the plan, by address
    std::vector<Step*> adams;
    for (Step& s : plan.steps)
    {
        if (s.kind == Step::ADAM)
            adams.push_back(&s);
        for (Step& g : s.group)
            if (s.kind == Step::ADAM_MULTI)
                adams.push_back(&g);
    }
    for (Step& s : plan.steps)
    {
        rt::Node* sum = s.kind == Step::ACT_BIAS_GRAD ? s.sum
                        : s.kind == Step::NODE && s.node->type == rt::Node::OP_MAT_SUM_COLS ? s.node : nullptr;
        if (!sum || keep.count(sum->out1))
            continue;
        const dbl_t* db = sum->out1;
        // every reader must be a gradient slot of an optimiser step
        bool ok = true;
        std::vector<std::pair<Step*, int>> slots;
        for (Step& other : plan.steps)
        {
            if (&other == &s || other.kind == Step::ADAM || other.kind == Step::ADAM_MULTI)
                continue;
            std::unordered_set<const dbl_t*> touched;
            tensors_of(other, touched);
            for (const Step& g : other.group)
                tensors_of(g, touched);
            if (touched.count(db))
                ok = false;
        }
        for (Step* a : adams)
        {
            const dbl_t* g1 = a->add ? a->add->in1 : a->m1->in1;
            const dbl_t* g2 = a->add && !a->grad_sum ? a->add->in2 : nullptr;
            if (g1 == db) slots.push_back({a, 0});
            if (g2 == db) slots.push_back({a, 1});
            // anything else of that step touching the tensor (its variable, a moment) rules it out
            for (const dbl_t* t : {(const dbl_t*)a->node->out1, (const dbl_t*)a->m1->out1, (const dbl_t*)a->m2->out1})
                if (t == db)
                    ok = false;
        }
        if (!ok || slots.empty())
            continue;
        // a stand-alone step without an `add` goes through dh_adam_step, which takes plain gradients
        for (auto& sl : slots)
            for (Step& top : plan.steps)
                if (&top == sl.first && top.kind == Step::ADAM && !top.add)
                    ok = false;
        if (!ok)
            continue;
        std::size_t nparts = dh_bias_grad_part_count(sum->len1, sum->len2);
        const dbl_t* sums = nullptr;
        if (nparts >= 2)
            sums = s.parts = parts_buffer(db, nparts * sum->len2);
        else if (s.kind == Step::NODE && sum->len1 >= 2 && sum->len1 <= 256 && written_once(plan, sum->in1))
        {
            // A matrix of few rows (the dense head's [batch x 1] logit gradients) is its own list of
            // row-range sums, one row each: the column-sum launches (two one-workgroup kernels, ~4.6 us
            // each whatever they do) go away and the optimiser launch adds the rows up.  The matrix is
            // written by one step only, so it still holds these values when the optimiser runs.
            s.rows_as_parts = true;
            sums = sum->in1;
            nparts = sum->len1;
        }
        else
            continue;
        for (auto& sl : slots)
        {
            sl.first->g_parts[sl.second] = sums;
            sl.first->g_nparts[sl.second] = nparts;
        }
    }
}

// ---- paired convolutions ---------------------------------------------------------------------------
// The discriminator runs twice per optimiser step, on the real and on the generated batch, with the
// same filters (dcgan/main.cu:304-307).  Two steps that are the same convolution with the same
// filter on independent activations are issued as ONE launch (dh_conv2d_*_pair): at batch 64 that
// halves the number of k splits a launch needs.  Two filter gradients whose sum is all the
// optimiser reads become one contraction over both.  The plan is re-ordered for this (the towers are
// interleaved layer by layer); every step still runs after the steps that produce its inputs.
struct ConvCall
{
    int kind = -1;            // 0 forward, 1 input gradient / transpose forward, 2 filter gradient,
                              // 3 tr(a) * b of a dense layer (g.N, g.H, g.W hold the product's m, n, p)
    ConvGeom g{};
    const dbl_t* a = nullptr;     // gathered activations (x, dy, x)
    const dbl_t* b = nullptr;     // filter (forward, input gradient) or dy (filter gradient)
    dbl_t* out = nullptr;
    const dbl_t* bias = nullptr;
    int act = DH_ACT_NONE;
    float alpha = 0.f;
};

bool conv_call_of(const Step& s, ConvCall& c)
{
    if (s.kind != Step::NODE && s.kind != Step::CONV_EPILOGUE)
        return false;
    if (s.kind == Step::NODE && s.act_ref)
        return false;
    const rt::Node* n = s.node;
    switch (n->type)
    {
    case rt::Node::OP_CONV2D: c.kind = 0; c.g = geom_conv2d(n); c.a = n->in1; c.b = n->in2; break;
    case rt::Node::OP_CONV2D_TRANSPOSE_INPUT_GRAD: c.kind = 0; c.g = geom_transpose_input_grad(n); c.a = n->in1; c.b = n->in2; break;
    case rt::Node::OP_CONV2D_INPUT_GRAD: c.kind = 1; c.g = geom_input_grad(n); c.a = n->in1; c.b = n->in2; break;
    case rt::Node::OP_CONV2D_TRANSPOSE: c.kind = 1; c.g = geom_transpose(n); c.a = n->in1; c.b = n->in2; break;
    case rt::Node::OP_CONV2D_KERNEL_GRAD: c.kind = 2; c.g = geom_kernel_grad(n); c.a = n->in2; c.b = n->in1; break;
    case rt::Node::OP_CONV2D_TRANSPOSE_KERNEL_GRAD: c.kind = 2; c.g = geom_transpose_kernel_grad(n); c.a = n->in1; c.b = n->in2; break;
    case rt::Node::OP_TMAT_MAT_MUL:
        if (s.kind != Step::NODE)
            return false;
        c.kind = 3; c.g = ConvGeom{}; c.g.N = (int)n->len1; c.g.H = (int)n->len2; c.g.W = (int)n->len3; c.a = n->in1; c.b = n->in2;
        break;
    default: return false;
    }
    c.out = n->out1;
    if (s.kind == Step::CONV_EPILOGUE)
    {
        if (c.kind == 2)
            return false;
        c.bias = s.bias ? s.bias->in2 : nullptr;
        c.act = s.act ? act_code(s.act) : DH_ACT_NONE;
        c.alpha = s.act ? s.act->alpha_leaky : 0.f;
        c.out = s.act ? s.act->out1 : s.bias->out1;
    }
    return true;
}

// What dh_conv2d_*_pair accepts: 16-byte chunks everywhere and operands below 2 GiB.
bool pairable(const ConvCall& c)
{
    const ConvGeom& g = c.g;
    if (c.kind == 3)
        return dh_gemm_tn_pair_supported((std::size_t)g.N, (std::size_t)g.H, (std::size_t)g.W) == 1;
    auto aligned = [](const void* q) { return (reinterpret_cast<std::uintptr_t>(q) & 15) == 0; };
    const double in_bytes = 4.0 * g.N * g.H * g.W * g.C, out_bytes = 4.0 * g.N * g.Ho * g.Wo * g.O;
    const double k_bytes = 4.0 * g.kh * g.kw * g.C * g.O, lim = 2147483648.0;
    // the paired launches need the buffer-load kernel, whose k-slabs of 16 must not straddle filter taps
    const bool tapwise = c.kind == 0 ? g.C % 16 == 0 : c.kind == 1 ? g.O % 16 == 0 : true;
    const bool sizes_ok = in_bytes < lim && out_bytes < lim && k_bytes < lim && aligned(c.a) && aligned(c.b) &&
                          aligned(c.out) && aligned(c.bias);
    // the forward product from a thin input (the image layer) and its filter gradient have paired kernels of their own
    if (c.kind == 0 && sizes_ok && g.C % 16 != 0 &&
        dh_conv2d_fwd_pair_supported(g.N, g.H, g.W, g.C, g.kh, g.kw, g.O, g.sh, g.sw, g.pt, g.pl, g.Ho, g.Wo) == 1)
        return true;
    if (c.kind == 2 && sizes_ok &&
        dh_conv2d_dk_pair_supported(g.N, g.H, g.W, g.C, g.Ho, g.Wo, g.O, g.kh, g.kw, g.sh, g.sw) == 1)
        return true;
    return tapwise && g.C % 4 == 0 && g.O % 4 == 0 && sizes_ok;
}

bool same_call(const ConvCall& x, const ConvCall& y)
{
    const ConvGeom &g = x.g, &h = y.g;
    const bool geom = g.N == h.N && g.H == h.H && g.W == h.W && g.C == h.C && g.Ho == h.Ho && g.Wo == h.Wo && g.O == h.O &&
                      g.kh == h.kh && g.kw == h.kw && g.sh == h.sh && g.sw == h.sw && g.pt == h.pt && g.pl == h.pl;
    if (!geom || x.kind != y.kind)
        return false;
    if (x.kind >= 2)
        return true;
    return x.b == y.b && x.bias == y.bias && x.act == y.act && x.alpha == y.alpha;
}

bool writes_in_place(const Step& s)
{
    if (s.kind == Step::ADAM || s.kind == Step::ADAM_MULTI)
        return true;
    const int t = s.node->type;
    return t == rt::Node::OP_UPDATE || t == rt::Node::OP_MOMENT_UPDATE || t == rt::Node::OP_MOMENT_UPDATE2 ||
           t == rt::Node::OP_ADAM_UPDATE;
}

void outputs_of(const Step& s, std::vector<const dbl_t*>& out)
{
    for (const rt::Node* n : {s.node, s.bias, s.act, s.sum, s.loss, s.node2, s.loss2,
                              s.kind == Step::SCE_HEAD ? s.add : nullptr})
        if (n && n->out1)
            out.push_back(n->out1);
}

void inputs_of(const Step& s, std::vector<const dbl_t*>& in)
{
    std::vector<const dbl_t*> outs;
    outputs_of(s, outs);
    auto add = [&](const dbl_t* t) {
        if (t && std::find(outs.begin(), outs.end(), t) == outs.end() && std::find(in.begin(), in.end(), t) == in.end())
            in.push_back(t);
    };
    add(s.act_ref);
    for (const rt::Node* n : nodes_of(s))
        if (n)
        {
            add(n->in1);
            add(n->in2);
            add(n->in3);
        }
    for (const Step& g : s.group)
        inputs_of(g, in);
}

void pair_convolutions(Plan& plan, const Keep& keep)
{
    std::vector<Step>& st = plan.steps;
    int n = 0;   // the steps before the first one that writes a variable in place may be re-ordered
    while (n < (int)st.size() && !writes_in_place(st[n]))
        ++n;
    if (n < 2)
        return;
    // who produces what, who depends (transitively) on whom, how often a tensor is read
    std::unordered_map<const dbl_t*, int> producer;
    std::unordered_map<const dbl_t*, int> reads;
    std::vector<std::vector<int>> deps(n);
    std::vector<std::vector<char>> reach(n, std::vector<char>(n, 0));
    for (int i = 0; i < (int)st.size(); ++i)
    {
        std::vector<const dbl_t*> in, out;
        inputs_of(st[i], in);
        for (const dbl_t* t : in)
            ++reads[t];
        if (i >= n)
            continue;
        for (const dbl_t* t : in)
        {
            auto f = producer.find(t);
            if (f == producer.end())
                continue;
            deps[i].push_back(f->second);
            reach[i][f->second] = 1;
            for (int q = 0; q < n; ++q)
                if (reach[f->second][q])
                    reach[i][q] = 1;
        }
        outputs_of(st[i], out);
        for (const dbl_t* t : out)
            producer[t] = i;
    }
    std::vector<ConvCall> call(n);
    std::vector<char> is_conv(n, 0);
    for (int i = 0; i < n; ++i)
        is_conv[i] = conv_call_of(st[i], call[i]) && pairable(call[i]);
    std::vector<int> partner(n, -1);
    // forward and input-gradient products with the same filter and epilogue
    for (int i = 0; i < n; ++i)
    {
        if (!is_conv[i] || call[i].kind >= 2 || partner[i] >= 0)
            continue;
        for (int j = i + 1; j < n; ++j)
            if (is_conv[j] && partner[j] < 0 && same_call(call[i], call[j]) && !reach[j][i])
            {
                partner[i] = j;
                partner[j] = i;
                break;
            }
    }
    // filter gradients that only meet in the sum an optimiser step reads
    std::vector<std::pair<int, int>> dk_pairs;   // (producer of add->in1, producer of add->in2)
    auto consider = [&](Step& adam) {
        if (adam.kind != Step::ADAM || !adam.add)
            return;
        auto pa = producer.find(adam.add->in1), pb = producer.find(adam.add->in2);
        if (pa == producer.end() || pb == producer.end() || pa->second == pb->second)
            return;
        const int a = pa->second, b = pb->second;
        if (!is_conv[a] || !is_conv[b] || call[a].kind < 2 || !same_call(call[a], call[b]) || partner[a] >= 0 ||
            partner[b] >= 0 || call[a].out != adam.add->in1 || call[b].out != adam.add->in2 ||
            reads[adam.add->in1] != 1 || reads[adam.add->in2] != 1 || keep.count(adam.add->in1) || keep.count(adam.add->in2))
            return;
        partner[a] = b;
        partner[b] = a;
        dk_pairs.push_back({a, b});
        adam.grad_sum = adam.add->in1;
    };
    for (int i = n; i < (int)st.size(); ++i)
    {
        consider(st[i]);
        for (Step& g : st[i].group)
            consider(g);
    }
    // two loss-plus-gradient steps whose losses an `add` joins: one launch for the three (the discriminator's
    // loss on the real and on the generated batch, dcgan/main.cu:304-307)
    std::vector<int> joined(n, -1);       // the `add` step of a pair of SCE_HEAD steps (at both members), -1 otherwise
    for (int k = 0; k < n; ++k)
    {
        const Step& add = st[k];
        if (add.kind != Step::NODE || add.node->type != rt::Node::OP_ADD || add.node->len1 != 1)
            continue;
        auto pa = producer.find(add.node->in1), pb = producer.find(add.node->in2);
        if (pa == producer.end() || pb == producer.end() || pa->second == pb->second)
            continue;
        const int a = pa->second, b = pb->second;
        if (st[a].kind != Step::SCE_HEAD || st[b].kind != Step::SCE_HEAD || st[a].node2 || st[b].node2 ||
            partner[a] >= 0 || partner[b] >= 0 || st[a].loss->out1 != add.node->in1 || st[b].loss->out1 != add.node->in2 ||
            st[a].node->len1 != st[b].node->len1)
            continue;
        partner[a] = b;
        partner[b] = a;
        joined[a] = joined[b] = k;
    }
    bool any = false;
    for (int i = 0; i < n; ++i)
        any = any || partner[i] >= 0;
    if (!any)
        return;
    // merge each pair into one node (named after its first member) and sort again: always the ready
    // node that stood first in the old order
    std::vector<int> node_of(n);
    for (int i = 0; i < n; ++i)
        node_of[i] = partner[i] >= 0 && partner[i] < i ? partner[i] : i;
    for (int i = 0; i < n; ++i)
        if (joined[i] >= 0)
            node_of[joined[i]] = node_of[i];
    std::vector<std::vector<int>> succ(n);
    std::vector<int> waiting(n, 0);
    for (int i = 0; i < n; ++i)
        for (int d : deps[i])
            if (node_of[d] != node_of[i])
            {
                succ[node_of[d]].push_back(node_of[i]);
                ++waiting[node_of[i]];
            }
    std::vector<Step> order;
    std::vector<char> done(n, 0);
    int nodes = 0, emitted = 0;
    for (int i = 0; i < n; ++i)
        nodes += node_of[i] == i;
    while (emitted < nodes)
    {
        int pick = -1;
        for (int i = 0; i < n && pick < 0; ++i)
            if (node_of[i] == i && !done[i] && waiting[i] == 0)
                pick = i;
        if (pick < 0)
        {
            // the merged graph has a cycle: leave the plan as it was
            for (Step& s : st)
            {
                s.grad_sum = nullptr;
                for (Step& g : s.group)
                    g.grad_sum = nullptr;
            }
            return;
        }
        done[pick] = 1;
        ++emitted;
        for (int v : succ[pick])
            --waiting[v];
        if (partner[pick] < 0)
            order.push_back(st[pick]);
        else if (joined[pick] >= 0)
        {
            // in the order of the `add` node's operands
            Step both = st[pick];
            const Step& other = st[partner[pick]];
            both.node2 = other.node;
            both.loss2 = other.loss;
            both.add = st[joined[pick]].node;
            order.push_back(both);
        }
        else
        {
            int first = pick, second = partner[pick];
            for (const auto& dk : dk_pairs)   // the contraction is written where the optimiser expects the sum
                if ((dk.first == first && dk.second == second) || (dk.first == second && dk.second == first))
                {
                    first = dk.first;
                    second = dk.second;
                }
            Step pair;
            pair.kind = Step::CONV_PAIR;
            pair.node = st[first].node;
            pair.group = {st[first], st[second]};
            order.push_back(pair);
        }
    }
    for (int i = n; i < (int)st.size(); ++i)
        order.push_back(st[i]);
    st.swap(order);
}

Plan make_plan(const std::vector<rt::Node*>& nodes, const Keep& keep, bool fuse)
{
    Plan plan;
    if (!fuse)
    {
        for (rt::Node* n : nodes)
        {
            Step s;
            s.node = n;
            plan.steps.push_back(s);
        }
        return plan;
    }
    Readers readers(nodes);
    std::unordered_set<rt::Node*> absorbed;
    // activation output that replaces a pre-activation tensor which is no longer materialised
    std::unordered_map<const dbl_t*, const dbl_t*> z_alias;
    std::unordered_map<rt::Node*, Step> fused_at;  // fused step keyed by the LAST node it replaces

    // the one instruction of the list that reads t
    auto sole_reader = [&](const dbl_t* t, rt::Node* who) {
        const auto& r = readers.of(t);
        return r.size() == 1 && r[0] == who;
    };
    // ... and the caller does not read it either: t need not exist after the run
    auto only_reader = [&](const dbl_t* t, rt::Node* who) { return !keep.count(t) && sole_reader(t, who); };

    // Whether an activation node may be folded into the launch that produces its input z: z is read only by
    // that activation and by gradient nodes that can take the activation's OUTPUT instead (same sign for
    // relu and for leaky with alpha > 0), and the caller does not ask for z itself.
    auto foldable_activation = [&](const dbl_t* z) -> rt::Node* {
        if (keep.count(z))
            return nullptr;
        rt::Node* act = nullptr;
        for (rt::Node* r : readers.of(z))
        {
            const int code = act_code(r);
            if (code >= 0 && r->in1 == z && !act)
                act = r;
            else if ((r->type == rt::Node::OP_RELU_GRAD || r->type == rt::Node::OP_LEAKY_RELU_GRAD) && r->in1 == z &&
                     r->in2 != z)
                ;  // redirected to the activation's output
            else
                return nullptr;
        }
        if (!act)
            return nullptr;
        const int code = act_code(act);
        for (rt::Node* r : readers.of(z))
        {
            if (r == act)
                continue;
            if (r->type == rt::Node::OP_RELU_GRAD && code != DH_ACT_RELU)
                return nullptr;
            if (r->type == rt::Node::OP_LEAKY_RELU_GRAD && !(code == DH_ACT_LEAKY && act->alpha_leaky > 0.f))
                return nullptr;
        }
        return act;
    };

    for (rt::Node* n : nodes)
    {
        if (absorbed.count(n))
            continue;
        if (n->type == rt::Node::OP_MAT_MUL_ADD)
        {
            // dense layer: mat_mul_add -> activation in the product's write-out
            rt::Node* act = foldable_activation(n->out1);
            if (!act || absorbed.count(act))
                continue;
            Step s;
            s.kind = Step::DENSE_EPILOGUE;
            s.node = n;
            s.act = act;
            absorbed.insert(act);
            z_alias[n->out1] = act->out1;
            fused_at[act] = s;
            continue;
        }
        if (is_conv_like(n))
        {
            // conv -> mat_rvect_add(conv_out, b) [-> activation(z)]
            rt::Node* bias = nullptr;
            for (rt::Node* r : readers.of(n->out1))
                if (r->type == rt::Node::OP_MAT_RVECT_ADD && r->in1 == n->out1)
                    bias = r;
            if (!bias || !only_reader(n->out1, bias))
                continue;
            Step s;
            s.kind = Step::CONV_EPILOGUE;
            s.node = n;
            s.bias = bias;
            absorbed.insert(bias);
            rt::Node* last = bias;
            if (rt::Node* act = foldable_activation(bias->out1))
            {
                s.act = act;
                absorbed.insert(act);
                z_alias[bias->out1] = act->out1;
                last = act;
            }
            fused_at[last] = s;
        }
    }
    // activation gradient -> mat_sum_cols, and the three Adam nodes of a variable
    for (rt::Node* n : nodes)
    {
        if (absorbed.count(n))
            continue;
        const bool act_grad = n->type == rt::Node::OP_RELU_GRAD || n->type == rt::Node::OP_LEAKY_RELU_GRAD ||
                              n->type == rt::Node::OP_TANH_GRAD;
        if (act_grad)
        {
            rt::Node* sum = nullptr;
            for (rt::Node* r : readers.of(n->out1))
                if (r->type == rt::Node::OP_MAT_SUM_COLS && !absorbed.count(r) && r->len1 * r->len2 == n->len1)
                    sum = r;
            if (sum)
            {
                Step s;
                s.kind = Step::ACT_BIAS_GRAD;
                s.node = n;
                s.sum = sum;
                absorbed.insert(n);
                absorbed.insert(sum);
                // emitted where the gradient node stood: dz feeds the dk / dx nodes that follow it
                fused_at[n] = s;
            }
        }
        if (n->type == rt::Node::OP_ADAM_UPDATE)
        {
            rt::Node *m1 = nullptr, *m2 = nullptr;
            for (rt::Node* p : n->preds)
            {
                if (p->type == rt::Node::OP_MOMENT_UPDATE && p->out1 == n->in1) m1 = p;
                if (p->type == rt::Node::OP_MOMENT_UPDATE2 && p->out1 == n->in2) m2 = p;
            }
            if (m1 && m2 && m1->in1 == m2->in1 && m1->len1 == n->len1 && m2->len1 == n->len1 &&
                !absorbed.count(m1) && !absorbed.count(m2) && sole_reader(m1->out1, n) && sole_reader(m2->out1, n))
            {
                // (the single pass writes both moments and the variable: nothing the caller could read is lost)
                Step s;
                s.kind = Step::ADAM;
                s.node = n;
                s.m1 = m1;
                s.m2 = m2;
                absorbed.insert(m1);
                absorbed.insert(m2);
                absorbed.insert(n);
                // gradient = add(a, b) read by nothing but these two moment updates: summed in the kernel
                for (rt::Node* q : nodes)
                    if (q->type == rt::Node::OP_ADD && q->out1 == m1->in1 && !absorbed.count(q) && !keep.count(q->out1) &&
                        q->len1 == n->len1)
                    {
                        const auto& rd = readers.of(q->out1);
                        bool only_moments = !rd.empty();
                        for (rt::Node* r : rd)
                            if (r != m1 && r != m2)
                                only_moments = false;
                        if (only_moments)
                        {
                            s.add = q;
                            absorbed.insert(q);
                        }
                    }
                fused_at[n] = s;
            }
        }
    }
    // sigmoid cross-entropy: the loss node and its gradient node on the same labels and logits become one
    // launch, issued where the first of the two stood (both outputs are still written)
    for (rt::Node* n : nodes)
    {
        if (n->type != rt::Node::OP_SIGMOID_CROSS_ENTROPY_GRAD || absorbed.count(n))
            continue;
        rt::Node* loss = nullptr;
        for (rt::Node* r : readers.of(n->in2))
            if (r->type == rt::Node::OP_SIGMOID_CROSS_ENTROPY && r->in1 == n->in1 && r->in2 == n->in2 && r->len1 == n->len1 &&
                !absorbed.count(r))
                loss = r;
        if (!loss)
            continue;
        Step s;
        s.kind = Step::SCE_HEAD;
        s.node = n;
        s.loss = loss;
        absorbed.insert(n);
        absorbed.insert(loss);
        rt::Node* first = n;
        for (rt::Node* q : nodes)
            if (q == n || q == loss)
            {
                first = q;
                break;
            }
        fused_at[first] = s;
    }
    for (rt::Node* n : nodes)
    {
        auto f = fused_at.find(n);
        if (f != fused_at.end())
        {
            Step s = f->second;
            if (s.kind == Step::ACT_BIAS_GRAD)
            {
                auto a = z_alias.find(s.node->in1);
                s.act_ref = a == z_alias.end() ? s.node->in1 : a->second;
            }
            plan.steps.push_back(s);
            continue;
        }
        if (absorbed.count(n))
            continue;
        // a product whose epilogue was fused is emitted at the position of the epilogue's last node
        bool conv_deferred = false;
        for (auto& kv : fused_at)
            if ((kv.second.kind == Step::CONV_EPILOGUE || kv.second.kind == Step::DENSE_EPILOGUE) && kv.second.node == n)
                conv_deferred = true;
        if (conv_deferred)
            continue;
        Step s;
        s.node = n;
        auto a = (n->type == rt::Node::OP_RELU_GRAD || n->type == rt::Node::OP_LEAKY_RELU_GRAD)
                     ? z_alias.find(n->in1)
                     : z_alias.end();
        s.act_ref = a == z_alias.end() ? nullptr : a->second;
        plan.steps.push_back(s);
    }
    gather_adam_steps(plan);
    if (g_pairing)
        pair_convolutions(plan, keep);
    defer_bias_sums(plan, keep);
    if (std::getenv("DCGAN_HIP_PLAN_DUMP"))
    {
        // the launches a run turns into, for inspection
        static const char* kinds[] = {"node", "conv+epilogue", "act-grad+bias-grad", "adam", "adam-multi", "pair",
                                      "dense+activation", "loss+gradient"};
        std::fprintf(stderr, "plan of %zu nodes -> %zu steps\n", nodes.size(), plan.steps.size());
        for (const Step& s : plan.steps)
            std::fprintf(stderr, "  %-20s %-32s len %zu\n", kinds[s.kind], op_name(s.node->type),
                         (std::size_t)s.node->len1);
    }
    return plan;
}

// The optimiser step of one variable as dh_adam_step_multi takes it: gradient g1 (+ g2 when the
// reference formed it with an `add` node that is not already folded into a paired filter gradient),
// either of them possibly as row-range sums (defer_bias_sums).
dh_adam_item adam_item(const Step& s, float lrt)
{
    rt::Node* a = s.node;
    const dbl_t* g1 = s.add ? s.add->in1 : s.m1->in1;
    const dbl_t* g2 = s.add && !s.grad_sum ? s.add->in2 : nullptr;
    dh_adam_item item{};
    item.p = a->out1; item.m = s.m1->out1; item.v = s.m2->out1;
    item.g1 = s.g_parts[0] ? s.g_parts[0] : g1;
    item.g2 = g2 ? (s.g_parts[1] ? s.g_parts[1] : g2) : nullptr;
    item.n = a->len1; item.lrt = lrt;
    item.g1_parts = s.g_parts[0] ? s.g_nparts[0] : 0;
    item.g2_parts = g2 && s.g_parts[1] ? s.g_nparts[1] : 0;
    return item;
}

void issue(const Step& s)
{
    switch (s.kind)
    {
    case Step::NODE:
    {
        rt::Node* n = s.node;
        if (s.act_ref)
        {
            // gradient of a fused activation: read the activation's output in place of z
            if (n->type == rt::Node::OP_RELU_GRAD)
                CK(dh_relu_grad(s.act_ref, n->in2, n->out1, n->len1, g_stream));
            else
                CK(dh_leaky_relu_grad(s.act_ref, n->in2, n->out1, n->cons1, n->len1, g_stream));
            return;
        }
        if (s.rows_as_parts)
            return;   // the optimiser launch reads the rows themselves
        if (s.parts)
        {
            // bias gradient left as row-range sums for the optimiser launch
            CK(dh_bias_grad_parts(n->in1, s.parts, n->len1, n->len2, g_stream));
            return;
        }
        kernel_f f = n->type >= 0 && n->type < 512 ? kernels_list[n->type] : nullptr;
        if (!f)
            throw std::runtime_error(std::string("hip backend: operator '") + op_name(n->type) +
                                     "' is not on the convolution path and has no HIP kernel");
        f(n);
        return;
    }
    case Step::CONV_EPILOGUE:
    {
        rt::Node* c = s.node;
        const dbl_t* bias = s.bias ? s.bias->in2 : nullptr;
        const int act = s.act ? act_code(s.act) : DH_ACT_NONE;
        const float alpha = s.act ? s.act->alpha_leaky : 0.f;
        dbl_t* out = s.act ? s.act->out1 : s.bias->out1;
        switch (c->type)
        {
        case rt::Node::OP_CONV2D: conv_fwd(geom_conv2d(c), c->in1, c->in2, out, bias, act, alpha); break;
        case rt::Node::OP_CONV2D_TRANSPOSE: conv_dx(geom_transpose(c), c->in1, c->in2, out, bias, act, alpha); break;
        case rt::Node::OP_CONV2D_INPUT_GRAD: conv_dx(geom_input_grad(c), c->in1, c->in2, out, bias, act, alpha); break;
        default: conv_fwd(geom_transpose_input_grad(c), c->in1, c->in2, out, bias, act, alpha); break;
        }
        return;
    }
    case Step::DENSE_EPILOGUE:
    {
        rt::Node* d = s.node;
        CK(dh_gemm_nn_act(d->in1, d->in2, d->in3, s.act->out1, d->len1, d->len2, d->len3, act_code(s.act), s.act->alpha_leaky,
                          g_stream));
        return;
    }
    case Step::SCE_HEAD:
    {
        rt::Node* g = s.node;
        if (s.node2)
            CK(dh_sigmoid_cross_entropy_head(g->in1, g->in2, s.loss->out1, g->out1, s.node2->in1, s.node2->in2, s.loss2->out1,
                                             s.node2->out1, s.add ? s.add->out1 : nullptr, g->len1, g_stream));
        else
            CK(dh_sigmoid_cross_entropy_head(g->in1, g->in2, s.loss->out1, g->out1, nullptr, nullptr, nullptr, nullptr, nullptr,
                                             g->len1, g_stream));
        return;
    }
    case Step::ACT_BIAS_GRAD:
    {
        rt::Node* g = s.node;
        const int act = g->type == rt::Node::OP_RELU_GRAD ? DH_ACT_RELU
                        : g->type == rt::Node::OP_LEAKY_RELU_GRAD ? DH_ACT_LEAKY : DH_ACT_TANH;
        if (s.parts)
            CK(dh_act_bias_grad_parts(s.act_ref, g->in2, g->out1, s.parts, s.sum->len1, s.sum->len2, act, g->cons1,
                                      g_stream));
        else
            CK(dh_act_bias_grad(s.act_ref, g->in2, g->out1, s.sum->out1, s.sum->len1, s.sum->len2, act, g->cons1,
                                g_stream));
        return;
    }
    case Step::ADAM:
    {
        rt::Node* a = s.node;
        const float lrt = adam_advance(a);
        if (s.add)
        {
            const dh_adam_item item = adam_item(s, lrt);
            CK(dh_adam_step_multi(&item, 1, s.m1->cons1, s.m1->cons2, s.m2->cons1, s.m2->cons2, a->cons4, g_stream));
        }
        else
            CK(dh_adam_step(a->out1, s.m1->out1, s.m2->out1, s.m1->in1, s.m1->cons1, s.m1->cons2, s.m2->cons1,
                            s.m2->cons2, lrt, a->cons4, a->len1, g_stream));
        return;
    }
    case Step::CONV_PAIR:
    {
        ConvCall a, b;
        conv_call_of(s.group[0], a);
        conv_call_of(s.group[1], b);
        const ConvGeom& g = a.g;
        if (a.kind == 0)
            CK(dh_conv2d_fwd_pair(a.a, b.a, a.b, a.out, b.out, g.N, g.H, g.W, g.C, g.kh, g.kw, g.O, g.sh, g.sw, g.pt, g.pl,
                                  g.Ho, g.Wo, a.bias, a.act, a.alpha, g_stream));
        else if (a.kind == 1)
            CK(dh_conv2d_dx_pair(a.a, b.a, a.b, a.out, b.out, g.N, g.Ho, g.Wo, g.O, g.kh, g.kw, g.C, g.sh, g.sw, g.pt, g.pl,
                                 g.H, g.W, a.bias, a.act, a.alpha, g_stream));
        else if (a.kind == 2)
            CK(dh_conv2d_dk_pair(a.a, a.b, b.a, b.b, a.out, g.N, g.H, g.W, g.C, g.Ho, g.Wo, g.O, g.kh, g.kw, g.sh, g.sw,
                                 g.pt, g.pl, g_stream));
        else
            CK(dh_gemm_tn_pair(a.a, a.b, b.a, b.b, a.out, (std::size_t)g.N, (std::size_t)g.H, (std::size_t)g.W, g_stream));
        return;
    }
    case Step::ADAM_MULTI:
    {
        std::vector<dh_adam_item> items;
        for (const Step& g : s.group)
        {
            rt::Node* a = g.node;
            const float lrt = adam_advance(a);
            items.push_back(adam_item(g, lrt));
        }
        const Step& f = s.group.front();
        CK(dh_adam_step_multi(items.data(), (int)items.size(), f.m1->cons1, f.m1->cons2, f.m2->cons1, f.m2->cons2,
                              f.node->cons4, g_stream));
        return;
    }
    }
}

// Plans are cached per instruction list (the lists of a training loop repeat every iteration).
struct PlanKey
{
    std::vector<rt::Node*> nodes;
    std::vector<const dbl_t*> keep;  // sorted
    bool keep_all;
    bool fuse;
    bool operator==(const PlanKey& o) const
    {
        return fuse == o.fuse && keep_all == o.keep_all && nodes == o.nodes && keep == o.keep;
    }
};
struct PlanKeyHash
{
    std::size_t operator()(const PlanKey& k) const
    {
        std::size_t h = (k.fuse ? 0x9e3779b97f4a7c15ull : 0) + (k.keep_all ? 1 : 0);
        for (rt::Node* n : k.nodes)
            h = (h ^ reinterpret_cast<std::size_t>(n)) * 0x100000001b3ull;
        for (const dbl_t* t : k.keep)
            h = (h ^ reinterpret_cast<std::size_t>(t)) * 0x100000001b3ull;
        return h;
    }
};
std::unordered_map<PlanKey, Plan, PlanKeyHash> g_plans;
Keep g_keep;

}  // namespace

void set_fusion(bool on)
{
    g_fusion = on ? 1 : 0;
}

void set_pairing(bool on)
{
    g_pairing = on;
}

bool fusion()
{
    if (g_fusion < 0)
    {
        const char* env = std::getenv("DCGAN_HIP_FUSE");
        g_fusion = env && !std::strcmp(env, "1") ? 1 : 0;
    }
    return g_fusion == 1;
}

namespace { bool g_sync_each_run = true; }
void set_sync_each_run(bool on) { g_sync_each_run = on; }
bool sync_each_run() { return g_sync_each_run; }

void* stream() { return g_stream; }   // hip_table.hh: the default stream

namespace { void flush_feeds(const Step* s); }

void synchronize()
{
    flush_feeds(nullptr);
    CK(dh_stream_sync(g_stream));
}

void set_protected_tensors(const std::vector<const dbl_t*>& tensors)
{
    g_keep.all = false;
    g_keep.set.clear();
    g_keep.set.insert(tensors.begin(), tensors.end());
}

void protect_all_tensors()
{
    g_keep.all = true;
    g_keep.set.clear();
}

// ---- inputs fed from host memory --------------------------------------------------------------
// The reference copies every fed input with a blocking cudaMemcpy in front of the run
// (src/ops/graph.cu:139-147), which first drains whatever is still executing and leaves the GPU idle
// while the host copies.  Here a fed input is only noted (feed); the run that follows stages and copies
// it, in stream order, right in front of the first step that touches the tensor, after the steps before
// it have been queued: the host stages the image batch of a discriminator step while the generator's
// forward pass runs.  (Sending the copy through a second stream with events either side was measured
// too: the two cross-stream waits per input cost more than the overlap of a 3 MB copy gains.)
namespace
{
struct Feed { dbl_t* begin; dbl_t* end; const dbl_t* src; };
std::vector<Feed> g_feeds;             // noted, not yet copied

bool node_touches(const rt::Node* n, const Feed& f)
{
    if (!n)
        return false;
    for (const dbl_t* t : {n->in1, n->in2, n->in3, (const dbl_t*)n->out1})
        if (t >= f.begin && t < f.end)
            return true;
    return false;
}

bool step_touches(const Step& s, const Feed& f)
{
    for (const rt::Node* n : nodes_of(s))
        if (node_touches(n, f))
            return true;
    if (s.act_ref >= f.begin && s.act_ref < f.end)
        return true;
    for (const Step& g : s.group)
        if (step_touches(g, f))
            return true;
    return false;
}

void copy_now(const Feed& f)
{
    CK(dh_memcpy_h2d_staged(f.begin, f.src, (std::size_t)(f.end - f.begin) * sizeof(dbl_t), g_stream));
}

// Copies the noted inputs that step `s` touches (all of them when s is null).
void flush_feeds(const Step* s)
{
    for (std::size_t i = 0; i < g_feeds.size();)
        if (!s || step_touches(*s, g_feeds[i]))
        {
            const Feed f = g_feeds[i];
            g_feeds.erase(g_feeds.begin() + (long)i);
            copy_now(f);
        }
        else
            ++i;
}
}  // namespace

void feed(dbl_t* dst, const dbl_t* src_host, std::size_t count)
{
    if (count == 0)
        return;
    // a second feed of the same tensor replaces the first
    for (std::size_t i = 0; i < g_feeds.size();)
        if (g_feeds[i].begin < dst + count && dst < g_feeds[i].end)
            g_feeds.erase(g_feeds.begin() + (long)i);
        else
            ++i;
    g_feeds.push_back(Feed{dst, dst + count, src_host});
}

void drop_feeds()
{
    g_feeds.clear();
}

void run_async(rt::NodesList& tasks)
{
    // the inputs noted for this run are borrowed host buffers: whatever happens, none outlives it
    struct DropFeeds { ~DropFeeds() { g_feeds.clear(); } } drop_feeds_on_exit;
    PlanKey key{tasks.nodes(), std::vector<const dbl_t*>(g_keep.set.begin(), g_keep.set.end()), g_keep.all, fusion()};
    std::sort(key.keep.begin(), key.keep.end());
    auto it = g_plans.find(key);
    if (it == g_plans.end())
        it = g_plans.emplace(key, make_plan(tasks.nodes(), g_keep, key.fuse)).first;
    for (const Step& s : it->second.steps)
    {
        if (!g_feeds.empty())
            flush_feeds(&s);
        issue(s);
    }
    // inputs the run did not touch: the caller's buffers are only borrowed until the run returns
    flush_feeds(nullptr);
    g_last_launches = 0;
    for (const Step& s : it->second.steps)
        g_last_launches += s.rows_as_parts ? 0 : 1;
}

int last_launch_count() { return g_last_launches; }

void run(rt::NodesList& tasks)
{
    run_async(tasks);
    synchronize();
}

void forget_plans()
{
    g_plans.clear();
    // the row-range-sum buffers belong to the plans that named them; blocks go back to the pool, which
    // hands them out again in stream order (see dh_pool_free), so no wait is needed here
    for (auto& kv : g_parts_pool)
        if (kv.second.first)
            CK(dh_pool_free(kv.second.first));
    g_parts_pool.clear();
}

}  // namespace hip
