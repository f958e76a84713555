// Model-building helpers on top of the operator graph (reference: src/api -- layers.hh:29-59,
// activ.hh:5-7, adam-optimizer.hh:7-23, initializer.hh, normal-initializer.hh, zero-initializer.hh).
#pragma once

#include <cstddef>
#include <cstdint>
#include <random>
#include <vector>

#include "ops.hh"

using activ_f = ops::Op* (*)(ops::Op*);

ops::Op* leaky_relu(ops::Op* x);  // alpha = 0.2
ops::Op* relu(ops::Op* x);
ops::Op* sigmoid(ops::Op* x);

class Initializer
{
public:
    virtual ~Initializer() = default;
    // [begin, end) is a tensor of the current program mode (device memory under RT_MODE=GPU).
    virtual void fill(dbl_t* begin, dbl_t* end) = 0;
};

class NormalInitializer : public Initializer
{
public:
    // The reference seeds from the clock (src/api/normal-initializer.cu:6-9); pass a seed to get
    // the same values on every run.
    NormalInitializer(dbl_t mean = 0, dbl_t sd = 1);
    NormalInitializer(dbl_t mean, dbl_t sd, std::uint64_t seed);
    void fill(dbl_t* begin, dbl_t* end) override;
    dbl_t next();

private:
    std::mt19937 engine_;
    std::normal_distribution<dbl_t> dist_;
};

class ZeroInitializer : public Initializer
{
public:
    void fill(dbl_t* begin, dbl_t* end) override;
};

struct DenseLayerData { ops::Op* w; ops::Op* b; ops::Op* z; };
struct Conv2DLayerData { ops::Op* w; ops::Op* b; ops::Op* z; };
struct Conv2DTransposeLayerData { ops::Op* w; ops::Op* b; ops::Op* z; };

// out = activ(input * w + b); w ~ N(0,1), b = 0 unless initialisers are given.
ops::Op* dense_layer(ops::Op* input, std::size_t in_size, std::size_t out_size, activ_f activ = nullptr,
                     Initializer* w_init = nullptr, Initializer* b_init = nullptr, DenseLayerData* tmp_data = nullptr);
// conv2d -> conv2d_bias_add -> activ, SAME padding.
ops::Op* conv2d_layer(ops::Op* input, std::size_t nb_filter, std::size_t* kernel_size, int* strides,
                      std::size_t* in_size, activ_f activ, Initializer* w_init, Initializer* b_init,
                      Conv2DLayerData* tmp_data);
// conv2d_transpose -> conv2d_bias_add -> activ; out_size = {out_height, out_width}.
ops::Op* conv2d_transpose_layer(ops::Op* input, std::size_t nb_filter, std::size_t* kernel_size,
                                std::size_t* out_size, int* strides, std::size_t* in_size, activ_f activ,
                                Initializer* w_init, Initializer* b_init, Conv2DTransposeLayerData* tmp_data);

class AdamOptimizer
{
public:
    AdamOptimizer(dbl_t learning_rate = 0.001, dbl_t beta1 = 0.9, dbl_t beta2 = 0.999, dbl_t epsilon = 1e-08);
    // One moment_update, moment_update2 and adam_update per variable, tied together by a seq
    // (src/api/adam-optimizer.cu:24-59).  The moments are non-trainable variables set to zero.
    ops::Op* minimize(ops::Op* loss, const std::vector<ops::Variable*>& vars = {});

private:
    dbl_t lr_, beta1_, beta2_, eps_;
};
