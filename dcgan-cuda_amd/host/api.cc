#include "api.hh"

#include <chrono>

#include "memory.hh"

ops::Op* leaky_relu(ops::Op* x) { return ops::OpsBuilder::instance().vect_relu_leaky(x); }
ops::Op* relu(ops::Op* x) { return ops::OpsBuilder::instance().vect_relu(x); }
ops::Op* sigmoid(ops::Op* x) { return ops::OpsBuilder::instance().vect_sigmoid(x); }

NormalInitializer::NormalInitializer(dbl_t mean, dbl_t sd)
    : engine_((std::mt19937::result_type)std::chrono::steady_clock::now().time_since_epoch().count()), dist_(mean, sd)
{
}

NormalInitializer::NormalInitializer(dbl_t mean, dbl_t sd, std::uint64_t seed)
    : engine_((std::mt19937::result_type)seed), dist_(mean, sd)
{
}

dbl_t NormalInitializer::next() { return dist_(engine_); }

void NormalInitializer::fill(dbl_t* begin, dbl_t* end)
{
    std::vector<dbl_t> host(end - begin);
    for (dbl_t& v : host)
        v = next();
    tensor_write(begin, end, host.data());
}

void ZeroInitializer::fill(dbl_t* begin, dbl_t* end) { tensor_fill(begin, end, 0); }

namespace
{
template <class Data>
ops::Op* finish_layer(ops::Op* z, ops::Op* w, ops::Op* b, activ_f activ, const char* activ_name, Data* tmp)
{
    ops::Op* out = z;
    if (activ)
    {
        out = activ(z);
        out->extend_name(activ_name);
    }
    if (tmp)
    {
        tmp->w = w;
        tmp->b = b;
        tmp->z = z;
    }
    return out;
}
}  // namespace

ops::Op* dense_layer(ops::Op* input, std::size_t in_size, std::size_t out_size, activ_f activ, Initializer* w_init,
                     Initializer* b_init, DenseLayerData* tmp_data)
{
    auto& builder = ops::OpsBuilder::instance();
    auto w = builder.variable(ops::Shape({int(in_size), int(out_size)}), true);
    w->extend_name("dense_w");
    auto b = builder.variable(ops::Shape({int(out_size)}), true);
    b->extend_name("dense_b");
    NormalInitializer w_default;
    ZeroInitializer b_default;
    (w_init ? w_init : &w_default)->fill(w->data_begin(), w->data_end());
    (b_init ? b_init : &b_default)->fill(b->data_begin(), b->data_end());
    return finish_layer(builder.mat_mul_add(input, w, b), w, b, activ, "dense_activ", tmp_data);
}

ops::Op* conv2d_layer(ops::Op* input, std::size_t nb_filter, std::size_t* kernel_size, int* strides,
                      std::size_t* in_size, activ_f activ, Initializer* w_init, Initializer* b_init,
                      Conv2DLayerData* tmp_data)
{
    auto& builder = ops::OpsBuilder::instance();
    auto w = builder.variable(ops::Shape({int(kernel_size[0]), int(kernel_size[1]), int(in_size[3]), int(nb_filter)}), true);
    w->extend_name("conv2d_w");
    auto b = builder.variable(ops::Shape({int(nb_filter)}), true);
    b->extend_name("conv2d_b");
    NormalInitializer fallback;
    (w_init ? w_init : &fallback)->fill(w->data_begin(), w->data_end());
    (b_init ? b_init : &fallback)->fill(b->data_begin(), b->data_end());
    ops::Op* conv = builder.conv2d(input, w, strides);
    return finish_layer(builder.conv2d_bias_add(conv, b), w, b, activ, "conv2d_activ", tmp_data);
}

ops::Op* conv2d_transpose_layer(ops::Op* input, std::size_t nb_filter, std::size_t* kernel_size, std::size_t* out_size,
                                int* strides, std::size_t* in_size, activ_f activ, Initializer* w_init,
                                Initializer* b_init, Conv2DTransposeLayerData* tmp_data)
{
    auto& builder = ops::OpsBuilder::instance();
    auto w = builder.variable(ops::Shape({int(kernel_size[0]), int(kernel_size[1]), int(nb_filter), int(in_size[3])}), true);
    w->extend_name("conv2d_transpose_w");
    auto b = builder.variable(ops::Shape({int(nb_filter)}), true);
    b->extend_name("conv2d_transpose_b");
    NormalInitializer fallback;
    (w_init ? w_init : &fallback)->fill(w->data_begin(), w->data_end());
    (b_init ? b_init : &fallback)->fill(b->data_begin(), b->data_end());
    const int out_shape[4] = {int(in_size[0]), int(out_size[0]), int(out_size[1]), int(nb_filter)};
    ops::Op* conv = builder.conv2d_transpose(input, w, out_shape, strides);
    return finish_layer(builder.conv2d_bias_add(conv, b), w, b, activ, "conv2d_transpose_activ", tmp_data);
}

AdamOptimizer::AdamOptimizer(dbl_t learning_rate, dbl_t beta1, dbl_t beta2, dbl_t epsilon)
    : lr_(learning_rate), beta1_(beta1), beta2_(beta2), eps_(epsilon)
{
}

ops::Op* AdamOptimizer::minimize(ops::Op* loss, const std::vector<ops::Variable*>& pvars)
{
    auto& graph = ops::Graph::instance();
    auto& builder = ops::OpsBuilder::instance();
    std::vector<ops::Variable*> vars = pvars.empty() ? graph.train_vars_get(loss) : pvars;
    std::vector<ops::Op*> updates;
    for (ops::Variable* v : vars)
    {
        ops::Op* grad = graph.gradient(loss, v);
        grad->extend_name("adam_grad");
        auto m = builder.variable(v->shape_get(), false);
        m->extend_name("adam_m");
        tensor_fill(m->data_begin(), m->data_end(), 0);
        auto s = builder.variable(v->shape_get(), false);
        s->extend_name("adam_v");
        tensor_fill(s->data_begin(), s->data_end(), 0);
        ops::Op* m_update = builder.moment_update(m, grad, beta1_, 1 - beta1_, false);
        ops::Op* s_update = builder.moment_update(s, grad, beta2_, 1 - beta2_, true);
        updates.push_back(builder.adam_update(v, m_update, s_update, lr_, beta1_, beta2_, eps_));
    }
    ops::Op* train = builder.seq(updates);
    train->extend_name("adam_train");
    return train;
}
