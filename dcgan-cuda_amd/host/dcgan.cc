#include "dcgan.hh"
#include "images.hh"
#include "npz.hh"

#include <cstddef>
#include <cstring>
#include <stdexcept>

#include "backend.hh"
#include "memory.hh"

namespace dcgan
{

namespace
{
constexpr int Z_DIM = 100;
int g_strides[2] = {2, 2};

ops::Op* transpose_block(ops::Op* input, const int* in_size, const int* out_size, bool use_activ,
                         Conv2DTransposeLayerData& data, Initializer& w_init)
{
    auto& builder = ops::OpsBuilder::instance();
    auto w = builder.variable(ops::Shape({5, 5, out_size[3], in_size[3]}), true);
    w->extend_name("conv2d_transpose_w");
    auto b = builder.variable(ops::Shape({out_size[3]}), true);
    b->extend_name("conv2d_transpose_b");
    ZeroInitializer zero;
    w_init.fill(w->data_begin(), w->data_end());
    zero.fill(b->data_begin(), b->data_end());
    ops::Op* z = builder.conv2d_bias_add(builder.conv2d_transpose(input, w, out_size, g_strides), b);
    data = {w, b, z};
    if (!use_activ)
        return z;
    ops::Op* out = relu(z);
    out->extend_name("conv2d_transpose_activ");
    return out;
}

ops::Op* conv_block(ops::Op* input, int in_channels, int nb_filter, Conv2DLayerData& data, bool reuse,
                    Initializer& w_init)
{
    auto& builder = ops::OpsBuilder::instance();
    if (!reuse)
    {
        auto w = builder.variable(ops::Shape({5, 5, in_channels, nb_filter}), true);
        w->extend_name("conv2d_w");
        auto b = builder.variable(ops::Shape({nb_filter}), true);
        b->extend_name("conv2d_b");
        ZeroInitializer zero;
        w_init.fill(w->data_begin(), w->data_end());
        zero.fill(b->data_begin(), b->data_end());
        data.w = w;
        data.b = b;
    }
    ops::Op* z = builder.conv2d_bias_add(builder.conv2d(input, data.w, g_strides), data.b);
    data.z = z;
    ops::Op* out = leaky_relu(z);
    out->extend_name("conv2d_activ");
    return out;
}

ops::Op* discriminator(Model& m, ops::Op* x, std::vector<ops::Op*>& nodes, Initializer& w_init)
{
    auto& builder = ops::OpsBuilder::instance();
    const bool reuse = !m.d_layers.empty();
    if (!reuse)
        m.d_layers.resize(4);
    const int chans[5] = {3, 64, 128, 256, 512};
    ops::Op* cur = x;
    for (int l = 0; l < 4; ++l)
    {
        cur = conv_block(cur, chans[l], chans[l + 1], m.d_layers[l], reuse, w_init);
        nodes.push_back(cur);
    }
    cur = builder.reshape(cur, ops::Shape({m.batch, 4 * 4 * 512}));
    if (!reuse)
    {
        auto w = builder.variable(ops::Shape({4 * 4 * 512, 1}), true);
        w->extend_name("dense_w");
        auto b = builder.variable(ops::Shape({1}), true);
        b->extend_name("dense_b");
        ZeroInitializer zero;
        w_init.fill(w->data_begin(), w->data_end());
        zero.fill(b->data_begin(), b->data_end());
        m.d_dense.w = w;
        m.d_dense.b = b;
    }
    ops::Op* logits = builder.mat_mul_add(cur, m.d_dense.w, m.d_dense.b);
    m.d_dense.z = logits;
    nodes.push_back(logits);
    return logits;
}
}  // namespace

Model* build(int batch, unsigned long long seed)
{
    auto& builder = ops::OpsBuilder::instance();
    auto* mp = new Model;
    Model& m = *mp;
    m.batch = batch;
    NormalInitializer w_init(0, 0.02, seed);

    m.z = builder.input(ops::Shape({batch, Z_DIM}));
    m.x = builder.input(ops::Shape({batch, 64, 64, 3}));

    // generator (dcgan/main.cu:89-120)
    ZeroInitializer zero;
    ops::Op* l0 = dense_layer(m.z, Z_DIM, 4 * 4 * 512, relu, &w_init, &zero, &m.g_dense);
    l0 = builder.reshape(l0, ops::Shape({batch, 4, 4, 512}));
    m.g_nodes.push_back(l0);
    const int sizes[5][4] = {{batch, 4, 4, 512}, {batch, 8, 8, 256}, {batch, 16, 16, 128}, {batch, 32, 32, 64},
                             {batch, 64, 64, 3}};
    m.g_layers.resize(4);
    ops::Op* cur = l0;
    for (int l = 0; l < 4; ++l)
    {
        cur = transpose_block(cur, sizes[l], sizes[l + 1], l < 3, m.g_layers[l], w_init);
        m.g_nodes.push_back(cur);
    }
    m.g_out = builder.vect_tanh(cur);

    // discriminator on generated and on real images, shared weights (dcgan/main.cu:217-249, :293-297)
    ops::Op* fake_logits = discriminator(m, m.g_out, m.d_fake_nodes, w_init);
    ops::Op* real_logits = discriminator(m, m.x, m.d_real_nodes, w_init);

    m.labels0 = builder.input(ops::Shape({batch, 1}));
    m.labels1 = builder.input(ops::Shape({batch, 1}));
    m.zeros.assign(batch, 0.f);
    m.ones.assign(batch, 1.f);

    // losses (dcgan/main.cu:304-307)
    m.g_loss = builder.sigmoid_cross_entropy(m.labels1, fake_logits);
    m.d_fake_loss = builder.sigmoid_cross_entropy(m.labels0, fake_logits);
    m.d_real_loss = builder.sigmoid_cross_entropy(m.labels1, real_logits);
    m.d_loss = builder.add(m.d_fake_loss, m.d_real_loss);
    m.y = builder.input(ops::Shape({batch, 1}));
    m.disc_loss = builder.sigmoid_cross_entropy(m.y, real_logits);

    for (auto& l : m.g_layers)
    {
        m.g_vars.push_back(dynamic_cast<ops::Variable*>(l.w));
        m.g_vars.push_back(dynamic_cast<ops::Variable*>(l.b));
    }
    m.g_vars.push_back(dynamic_cast<ops::Variable*>(m.g_dense.w));
    m.g_vars.push_back(dynamic_cast<ops::Variable*>(m.g_dense.b));
    for (auto& l : m.d_layers)
    {
        m.d_vars.push_back(dynamic_cast<ops::Variable*>(l.w));
        m.d_vars.push_back(dynamic_cast<ops::Variable*>(l.b));
    }
    m.d_vars.push_back(dynamic_cast<ops::Variable*>(m.d_dense.w));
    m.d_vars.push_back(dynamic_cast<ops::Variable*>(m.d_dense.b));

    // Adam(2e-4, 0.5) for each network (dcgan/main.cu:329-332)
    AdamOptimizer g_adam(0.0002, 0.5);
    m.g_opti = g_adam.minimize(m.g_loss, m.g_vars);
    AdamOptimizer d_adam(0.0002, 0.5);
    m.d_opti = d_adam.minimize(m.d_loss, m.d_vars);
    return mp;
}

}  // namespace dcgan

namespace
{
thread_local std::string g_error;

template <class F>
int guarded(F f)
{
    try
    {
        f();
        return 0;
    }
    catch (const std::exception& e)
    {
        g_error = e.what();
        return 1;
    }
}

dcgan::Model& M(void* p) { return *static_cast<dcgan::Model*>(p); }

ops::Variable* var_at(dcgan::Model& m, int i)
{
    const int ng = (int)m.g_vars.size();
    if (i < 0 || i >= ng + (int)m.d_vars.size())
        throw std::runtime_error("variable index out of range");
    return i < ng ? m.g_vars[i] : m.d_vars[i - ng];
}

void bind_labels(dcgan::Model& m)
{
    // the label inputs are constants: bound once, then resident
    auto& g = ops::Graph::instance();
    const ops::Shape s({m.batch, 1});
    g.run({m.labels0, m.labels1}, {{m.labels0, {m.zeros.data(), s}}, {m.labels1, {m.ones.data(), s}}}, {});
}

ops::Op* lookup(dcgan::Model& m, const std::string& what)
{
    auto& g = ops::Graph::instance();
    auto layer = [&](const std::string& prefix, std::vector<ops::Op*>& nodes, const char* last) -> ops::Op* {
        if (what == prefix + last)
            return nodes.back();
        for (std::size_t i = 0; i + 1 < nodes.size() || (i < nodes.size() && !*last); ++i)
            if (what == prefix + "l" + std::to_string(i))
                return nodes[i];
        return nullptr;
    };
    if (what == "g_out") return m.g_out;
    if (what == "g_loss") return m.g_loss;
    if (what == "d_loss") return m.d_loss;
    if (what == "d_fake_loss") return m.d_fake_loss;
    if (what == "d_real_loss") return m.d_real_loss;
    if (what == "disc_loss") return m.disc_loss;
    if (what.rfind("g_l", 0) == 0)
    {
        const int i = std::stoi(what.substr(3));
        return m.g_nodes.at(i);
    }
    if (ops::Op* o = layer("d_fake_", m.d_fake_nodes, "logits")) return o;
    if (ops::Op* o = layer("d_real_", m.d_real_nodes, "logits")) return o;
    if (what.rfind("grad:", 0) == 0)
    {
        const std::size_t c = what.find(':', 5);
        const std::string loss = what.substr(5, c - 5), target = what.substr(c + 1);
        ops::Op* l = loss == "g_loss" ? m.g_loss : loss == "d_loss" ? m.d_loss : loss == "disc_loss" ? m.disc_loss : nullptr;
        if (!l)
            throw std::runtime_error("unknown loss " + loss);
        if (target == "x_fake")
            return g.gradient(l, m.g_out);
        if (target == "x_real")
            return g.gradient(l, m.x);
        return g.gradient(l, var_at(m, std::stoi(target)));
    }
    throw std::runtime_error("unknown tensor " + what);
}
}  // namespace

extern "C" {

const char* dg_last_error(void) { return g_error.c_str(); }

void* dg_create(int batch, unsigned long long seed)
{
    dcgan::Model* m = nullptr;
    if (guarded([&] {
            m = dcgan::build(batch, seed);
            bind_labels(*m);
        }))
        return nullptr;
    return m;
}

void dg_destroy(void* model)
{
    guarded([&] {
        ops::Graph::instance().exit_graph();
        delete static_cast<dcgan::Model*>(model);
    });
}

void dg_set_fusion(int fuse)
{
    hip::set_fusion(fuse != 0);
    hip::forget_plans();
}

void dg_set_name_results(int on)
{
    ops::Graph::instance().name_results_set(on != 0);
    hip::forget_plans();
}

void dg_set_pairing(int on)
{
    hip::set_pairing(on != 0);
    hip::forget_plans();
}

int dg_num_vars(void* model) { return (int)(M(model).g_vars.size() + M(model).d_vars.size()); }

long dg_var_size(void* model, int index)
{
    long n = -1;
    guarded([&] { n = var_at(M(model), index)->shape_get().total(); });
    return n;
}

int dg_var_read(void* model, int index, float* host)
{
    return guarded([&] { var_at(M(model), index)->read(host); });
}

int dg_var_write(void* model, int index, const float* host)
{
    return guarded([&] { var_at(M(model), index)->write(host); });
}

int dg_set_inputs(void* model, const float* z_host, const float* x_host)
{
    return guarded([&] {
        dcgan::Model& m = M(model);
        std::map<ops::Input*, std::pair<const dbl_t*, ops::Shape>> in;
        std::vector<ops::Op*> targets;
        if (z_host)
        {
            in[m.z] = {z_host, ops::Shape({m.batch, 100})};
            targets.push_back(m.z);
        }
        if (x_host)
        {
            in[m.x] = {x_host, ops::Shape({m.batch, 64, 64, 3})};
            targets.push_back(m.x);
        }
        ops::Graph::instance().run(targets, in, {});
    });
}

namespace
{
std::map<ops::Input*, std::pair<const dbl_t*, ops::Shape>> fed(dcgan::Model& m, const float* z_host, const float* x_host)
{
    std::map<ops::Input*, std::pair<const dbl_t*, ops::Shape>> in;
    if (z_host)
        in[m.z] = {z_host, ops::Shape({m.batch, 100})};
    if (x_host)
        in[m.x] = {x_host, ops::Shape({m.batch, 64, 64, 3})};
    return in;
}
}  // namespace

int dg_d_step(void* model, float* d_loss) { return dg_d_step_fed(model, nullptr, nullptr, d_loss); }

int dg_d_step_fed(void* model, const float* z_host, const float* x_host, float* d_loss)
{
    return guarded([&] {
        dcgan::Model& m = M(model);
        hip::set_sync_each_run(d_loss != nullptr);
        ops::Graph::instance().run({m.d_opti, m.d_loss}, fed(m, z_host, x_host), {nullptr, d_loss});
        hip::set_sync_each_run(true);
    });
}

int dg_g_step(void* model, float* g_loss) { return dg_g_step_fed(model, nullptr, g_loss); }

int dg_g_step_fed(void* model, const float* z_host, float* g_loss)
{
    return guarded([&] {
        dcgan::Model& m = M(model);
        hip::set_sync_each_run(g_loss != nullptr);
        ops::Graph::instance().run({m.g_opti, m.g_loss}, fed(m, z_host, nullptr), {nullptr, g_loss});
        hip::set_sync_each_run(true);
    });
}

int dg_set_labels(void* model, const float* y_host)
{
    return guarded([&] {
        dcgan::Model& m = M(model);
        ops::Graph::instance().run({m.y}, {{m.y, {y_host, ops::Shape({m.batch, 1})}}}, {});
    });
}

int dg_disc_pass(void* model, float* loss)
{
    return guarded([&] {
        dcgan::Model& m = M(model);
        auto& g = ops::Graph::instance();
        if (m.disc_targets.empty())
        {
            m.disc_targets.push_back(m.disc_loss);
            for (ops::Variable* v : m.d_vars)
                m.disc_targets.push_back(g.gradient(m.disc_loss, v));
            m.disc_targets.push_back(g.gradient(m.disc_loss, m.x));
        }
        std::vector<dbl_t*> outs(m.disc_targets.size(), nullptr);
        outs[0] = loss;
        hip::set_sync_each_run(loss != nullptr);
        g.run(m.disc_targets, {}, outs);
        hip::set_sync_each_run(true);
    });
}

int dg_sync(void)
{
    return guarded([] {
        if (program_mode() == ProgramMode::GPU)
            hip::synchronize();
    });
}

int dg_generate(void* model, float* images_host)
{
    // images_host == nullptr: the images stay on the device and the run is not waited for
    return guarded([&] {
        hip::set_sync_each_run(images_host != nullptr);
        ops::Graph::instance().run({M(model).g_out}, {}, {images_host});
        hip::set_sync_each_run(true);
    });
}

int dg_eval(void* model, const char* what, float* host, long* count)
{
    return guarded([&] {
        ops::Op* op = lookup(M(model), what);
        if (count)
            *count = op->shape_get().total();
        if (host)
            ops::Graph::instance().run({op}, {}, {host});
    });
}

int dg_eval_many(void* model, const char* names, float** hosts, int count)
{
    return guarded([&] {
        std::vector<ops::Op*> targets;
        std::vector<dbl_t*> outs;
        const std::string all(names);
        std::size_t at = 0;
        while (at <= all.size() && (int)targets.size() < count)
        {
            std::size_t end = all.find(';', at);
            if (end == std::string::npos)
                end = all.size();
            targets.push_back(lookup(M(model), all.substr(at, end - at)));
            outs.push_back(hosts[targets.size() - 1]);
            at = end + 1;
        }
        if ((int)targets.size() != count)
            throw std::runtime_error("dg_eval_many: fewer names than count");
        ops::Graph::instance().run(targets, {}, outs);
    });
}

int dg_save_vars(void*, const char* path) { return guarded([&] { ops::Graph::instance().save_vars(path); }); }
int dg_load_vars(void*, const char* path) { return guarded([&] { ops::Graph::instance().load_vars(path); }); }
int dg_save_state(void*, const char* path) { return guarded([&] { ops::Graph::instance().save_state(path); }); }
int dg_load_state(void*, const char* path) { return guarded([&] { ops::Graph::instance().load_state(path); }); }

int dg_npz_inspect(const char* path, long* arrays, long* elements)
{
    return guarded([&] {
        const std::vector<npz::Array> all = npz::load(path);
        long n = 0;
        for (const npz::Array& a : all)
            n += (long)a.data.size();
        if (arrays)
            *arrays = (long)all.size();
        if (elements)
            *elements = n;
    });
}

int dg_images_normalize(const unsigned char* pix, long count, float* out)
{
    return guarded([&] { images::normalize(pix, (std::size_t)count, out); });
}

int dg_images_load(const char* dir, long idx_beg, long idx_end, float* out)
{
    return guarded([&] {
        const std::vector<dbl_t> batch = images::load(dir, (std::size_t)idx_beg, (std::size_t)idx_end);
        std::copy(batch.begin(), batch.end(), out);
    });
}

int dg_images_save_samples(const float* data, long width, long height, const char* path)
{
    return guarded([&] { images::save_samples(data, (std::size_t)width, (std::size_t)height, path); });
}

// sizeof(rt::Node) followed by the offset of every field a kernel-table entry reads, in declaration
// order: type, in1, in2, in3, out1, out2, cons1..4, len1..3, intconst, intconst2, sizes1..3,
// int_cons1, int_cons2, alpha_leaky.  Returns the number of values written (at most n).
#pragma GCC diagnostic push
#pragma GCC diagnostic ignored "-Winvalid-offsetof"
int dg_node_layout(unsigned long* out, int n)
{
    using N = rt::Node;
    const unsigned long v[] = {sizeof(N), offsetof(N, type), offsetof(N, in1), offsetof(N, in2), offsetof(N, in3),
                               offsetof(N, out1), offsetof(N, out2), offsetof(N, cons1), offsetof(N, cons2),
                               offsetof(N, cons3), offsetof(N, cons4), offsetof(N, len1), offsetof(N, len2),
                               offsetof(N, len3), offsetof(N, intconst), offsetof(N, intconst2), offsetof(N, sizes1),
                               offsetof(N, sizes2), offsetof(N, sizes3), offsetof(N, int_cons1), offsetof(N, int_cons2),
                               offsetof(N, alpha_leaky)};
    const int count = (int)(sizeof(v) / sizeof(v[0]));
    for (int i = 0; i < count && i < n; ++i)
        out[i] = v[i];
    return count < n ? count : n;
}
#pragma GCC diagnostic pop

int dg_last_launch_count(void*) { return hip::last_launch_count(); }

int dg_last_schedule_size(void*)
{
    return (int)ops::Graph::instance().last_schedule().size();
}

}
