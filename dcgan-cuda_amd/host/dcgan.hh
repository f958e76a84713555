// The DCGAN of the reference application (dcgan/main.cu:41-332) built on the operator graph, and a
// C facade over it for the benchmark and the parity tests.  64x64x3 images, z of dimension 100,
// 5x5 filters, stride 2, SAME padding.
//   generator      dense 100 -> 4*4*512 + relu, 4 x (conv2d_transpose + bias [+ relu]), tanh
//   discriminator  4 x (conv2d + bias + leaky_relu 0.2), dense 8192 -> 1; weights shared between
//                  the branch fed by the generator and the branch fed by real images
//   losses         sigmoid cross-entropy; d_loss = D(fake) vs 0 + D(real) vs 1; g_loss = D(fake) vs 1
//   optimiser      Adam(lr 2e-4, beta1 0.5, beta2 0.999, eps 1e-8) per network
#pragma once

#include <string>
#include <vector>

#include "api.hh"

namespace dcgan
{

struct Model
{
    int batch = 0;
    ops::Input *z = nullptr, *x = nullptr, *labels0 = nullptr, *labels1 = nullptr;
    DenseLayerData g_dense{};
    std::vector<Conv2DTransposeLayerData> g_layers;
    std::vector<ops::Op*> g_nodes;          // l0 .. l4 (pre-tanh)
    ops::Op* g_out = nullptr;
    DenseLayerData d_dense{};
    std::vector<Conv2DLayerData> d_layers;
    std::vector<ops::Op*> d_fake_nodes, d_real_nodes;  // l0 .. l3, logits
    ops::Op *g_loss = nullptr, *d_fake_loss = nullptr, *d_real_loss = nullptr, *d_loss = nullptr;
    std::vector<ops::Variable*> g_vars, d_vars;        // (w, b) per layer, dense last -- dcgan/main.cu:309-325
    ops::Op *g_opti = nullptr, *d_opti = nullptr;
    std::vector<dbl_t> ones, zeros;
    // The discriminator by itself on labelled images (tests/test_dcgan_discriminator.cu:49-136): labels y,
    // loss = sigmoid cross-entropy(y, D(x)) on the tower fed by x, and the pass's targets -- the loss, its
    // gradient for every discriminator variable and for the images themselves.
    ops::Input* y = nullptr;
    ops::Op* disc_loss = nullptr;
    std::vector<ops::Op*> disc_targets;
};

// Builds the whole graph (both networks, losses, gradients, Adam).  Weights ~ N(0, 0.02) from
// `seed`, biases zero.  One Model per process: the operator graph is a process-wide singleton.
Model* build(int batch, unsigned long long seed);

}  // namespace dcgan

extern "C" {
// Every function returns 0 on success; dg_last_error() describes the last failure.
const char* dg_last_error(void);
// RT_MODE must be set before the first call (GPU for the HIP backend).
void* dg_create(int batch, unsigned long long seed);
void dg_destroy(void* model);
// fuse != 0: run fused convolution epilogues, activation+bias gradients and single-pass Adam.
void dg_set_fusion(int fuse);
// on != 0 (the default): with fusion, same-filter convolutions of independent towers run as one paired launch.
void dg_set_pairing(int on);
// The discriminator alone (forward + backward, no optimiser): dg_set_labels binds the [batch, 1] labels,
// dg_disc_pass computes the loss, all ten parameter gradients and the gradient of the input images in one run
// (loss == NULL: nothing is read back and the run is not waited for).
int dg_set_labels(void* model, const float* y_host);
int dg_disc_pass(void* model, float* loss);
// on == 0: every run hands the backend its instruction list and nothing else, as the reference's Graph::run
// does (src/ops/graph.cu:194-200), so the planner keeps every intermediate tensor; on != 0 (the default): the
// run names the tensors it reads back and the others may be left out.
void dg_set_name_results(int on);
// Variables in the order g conv-transpose 1..4 (w,b), g dense (w,b), d conv 0..3 (w,b), d dense (w,b).
int dg_num_vars(void* model);
long dg_var_size(void* model, int index);
int dg_var_read(void* model, int index, float* host);
int dg_var_write(void* model, int index, const float* host);
// Copies one batch of z [batch,100] / images [batch,64,64,3] to the device-resident inputs.
int dg_set_inputs(void* model, const float* z_host, const float* x_host);
// One discriminator / generator Adam step on the resident inputs; loss may be NULL (then nothing
// is copied back and the call returns while the GPU is still running).
int dg_d_step(void* model, float* d_loss);
int dg_g_step(void* model, float* g_loss);
// The same with the inputs handed to the run itself, as the reference's training loop does
// (dcgan/main.cu:378-391: graph.run({opti, loss}, {{z, ...}, {x, ...}}, ...)); a NULL input stays as it is
// on the device.  The buffers are borrowed until the call returns.
int dg_d_step_fed(void* model, const float* z_host, const float* x_host, float* d_loss);
int dg_g_step_fed(void* model, const float* z_host, float* g_loss);
int dg_sync(void);
// Generator forward only: images [batch,64,64,3] to host.
int dg_generate(void* model, float* images_host);
// Evaluate a named tensor on the resident inputs WITHOUT applying an update and copy it to host:
//   "g_l0".."g_l4", "g_out", "d_fake_l0".."d_fake_l3", "d_fake_logits", "d_real_l0".., "d_real_logits",
//   "g_loss", "d_loss", "d_fake_loss", "d_real_loss",
//   "grad:g_loss:<var index>", "grad:d_loss:<var index>", "grad:g_loss:x_fake" (d g_loss / d g_out)
// Returns the number of elements through *count; host may be NULL to query the size only.
int dg_eval(void* model, const char* what, float* host, long* count);
// The same for `count` tensors named in one ';'-separated string, evaluated in ONE run of the graph
// (shared upstream tensors are computed once); hosts[i] receives the i-th tensor.
int dg_eval_many(void* model, const char* names, float** hosts, int count);
// Trainable variables to / from a file (numpy .npz when the path ends in ".npz"); the whole training
// state (all variables, Adam moments and step counters) as .npz.  The model argument is unused: the
// operator graph is a process-wide singleton.
int dg_save_vars(void* model, const char* path);
int dg_load_vars(void* model, const char* path);
int dg_save_state(void* model, const char* path);
int dg_load_state(void* model, const char* path);
// Reads a .npz archive with the reader behind dg_load_vars / dg_load_state and reports how many arrays
// and elements it holds; fails (with the reader's message) on anything it would refuse to load.
int dg_npz_inspect(const char* path, long* arrays, long* elements);
// Image helpers (host/images.hh): 8-bit pixels to [-1, 1]; images <dir>/<6-digit index>.ppm for
// idx_beg <= index < idx_end as one normalised batch; width x height generated images as one PPM mosaic.
int dg_images_normalize(const unsigned char* pix, long count, float* out);
int dg_images_load(const char* dir, long idx_beg, long idx_end, float* out);
int dg_images_save_samples(const float* data, long width, long height, const char* path);
// Layout of this library's rt::Node (size, then field offsets): equal to the reference's record
// (src/runtime/node.hh:215-242) field for field, which a test checks against a build of the reference.
int dg_node_layout(unsigned long* out, int n);
// Number of rt::Node instructions / fused launches of the last run.
int dg_last_schedule_size(void* model);
int dg_last_launch_count(void* model);
}
