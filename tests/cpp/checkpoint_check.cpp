// Host program for the checkpoint tests: builds a network through the adaptor, optionally trains it for two steps on the
// device, writes the reference's two text files, reads them into a second object, writes them again and compares - the
// files byte for byte, and with a device the inference outputs of both objects bit for bit.
// usage: checkpoint_check <dir> <kind> [device]      kinds: mlp, recurrent, normalised, residual
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iterator>
#include <string>
#include <vector>

#include "../../include/myea_nn_hip.hpp"

using namespace MyEA_HIP;

static std::string slurp(const std::string &path)
{
    std::ifstream f(path, std::ios::binary);
    return std::string((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
}

static unsigned long long rng_state = 0x2545F4914F6CDD1Dull;
static float rnd()   // xorshift, uniform in [-0.5, 0.5)
{
    rng_state ^= rng_state << 13; rng_state ^= rng_state >> 7; rng_state ^= rng_state << 17;
    return (float)((rng_state >> 40) & 0xFFFFFF) / 16777216.f - 0.5f;
}

static bool build(Neural_Network_HIP &nn, const std::string &kind, size_t B, size_t *T, size_t *n_in, size_t *n_out)
{
    if (!nn.Update__Batch_Size(B)) return false;
    if (kind == "mlp") {   // 12 -> 16 (renorm before, ReLU, Gaussian dropout) -> max pooling -> 10 (tanh, BN after, k-sparse) -> 5 softmax
        *T = 1; *n_in = 12; *n_out = 5;
        Layer_Parameters layers[5];
        for (auto &l : layers) l.type_layer = MYEA_LAYER_FULLY_CONNECTED;
        layers[0].unit_parameters[0] = 12; layers[1].unit_parameters[0] = 16; layers[3].unit_parameters[0] = 10; layers[4].unit_parameters[0] = 5;
        layers[2].type_layer = MYEA_LAYER_MAX_POOLING;
        layers[2].unit_parameters[0] = 3; layers[2].unit_parameters[1] = 2; layers[2].unit_parameters[2] = 1; layers[2].unit_parameters[3] = 1; layers[2].unit_parameters[4] = 1;
        if (!nn.Compile(5, *T, MYEA_NETWORK_FEEDFORWARD, layers)) return false;
        T_ gauss[2] = {0.2f, 0.f};
        if (!nn.Set__Layer_Activation_Function(1, MYEA_AF_RELU) || !nn.Set__Layer_Activation_Function(3, MYEA_AF_TANH) || !nn.Set__Layer_Activation_Function(4, MYEA_AF_SOFTMAX) ||
            !nn.Set__Layer_Normalization(1, MYEA_NORMALIZATION_BATCH_RENORMALIZATION, true) || !nn.Set__Layer_Normalization(3, MYEA_NORMALIZATION_BATCH_NORMALIZATION, false) ||
            !nn.Set__Dropout(1, MYEA_DROPOUT_GAUSSIAN, gauss) || !nn.Set__K_Sparsity(3, 4) || !nn.Set__Alpha_Sparsity(3, 2.f) || !nn.Set__Layer_Activation_Steepness(3, 0.75f)) return false;
        nn.Set__Loss_Function(MYEA_LOSS_CROSS_ENTROPY); nn.Set__Accuracy_Function(MYEA_ACCURACY_CROSS_ENTROPY); nn.Set__Optimizer_Function(MYEA_OPTIMIZER_AMSGRAD);
        nn.adam_learning_rate = 0.002f; nn.adam_beta1 = 0.85f; nn.regularization__weight_decay = 1e-4f; nn.batch_renormalization_r_correction_maximum = 1.5f;
        nn.batch_renormalization_d_correction_maximum = 0.25f; nn.normalization_momentum_average = 0.9f;
    } else if (kind == "recurrent") {   // 6 -> LSTM 4 blocks x 2 cells (zoneout) -> IndRNN-9 tanh (custom bounds) -> 9 linear, T = 4, one time delay
        *T = 4; *n_in = 6; *n_out = 3;
        Layer_Parameters layers[4];
        layers[0].type_layer = MYEA_LAYER_FULLY_CONNECTED; layers[0].unit_parameters[0] = 6;
        layers[1].type_layer = MYEA_LAYER_LSTM; layers[1].unit_parameters[0] = 4; layers[1].unit_parameters[1] = 2;
        layers[2].type_layer = MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT; layers[2].unit_parameters[0] = 9;
        layers[3].type_layer = MYEA_LAYER_FULLY_CONNECTED; layers[3].unit_parameters[0] = 9;
        if (!nn.Compile(4, *T, MYEA_NETWORK_RECURRENT, layers)) return false;
        *n_out = 9;
        T_ zone[2] = {0.1f, 0.05f};
        if (!nn.Set__Layer_Activation_Function(2, MYEA_AF_TANH) || !nn.Set__Regularization__Constraint_Recurrent_Weight(2, -0.5f, 0.75f) ||
            !nn.Set__Layer_Activation_Function(3, MYEA_AF_LINEAR) || !nn.Set__Dropout(1, MYEA_DROPOUT_ZONEOUT, zone) || !nn.Set__Number_Time_Delays(1)) return false;
        nn.Set__Loss_Function(MYEA_LOSS_MSE); nn.Set__Optimizer_Function(MYEA_OPTIMIZER_GD);
        nn.learning_rate = 0.02f; nn.learning_momentum = 0.5f; nn.use_Nesterov = true; nn.Set__Clip_Gradient(true); nn.clip_gradient = 2.5f;
        nn.use_Warm_Restarts = true; nn.warm_restarts_initial_maximum_learning_rate = nn.warm_restarts_maximum_learning_rate = 0.5f;
        nn.warm_restarts_initial_T_i = nn.warm_restarts_T_i = 8.f; nn.warm_restarts_multiplier = 3.f; nn.regularization__max_norm_constraints = 4.f;
    } else if (kind == "normalised") {   // 5 -> LSTM 6 blocks of one cell, batch renormalisation -> 6 linear, T = 3
        *T = 3; *n_in = 5; *n_out = 6;
        Layer_Parameters layers[3];
        layers[0].type_layer = MYEA_LAYER_FULLY_CONNECTED; layers[0].unit_parameters[0] = 5;
        layers[1].type_layer = MYEA_LAYER_LSTM; layers[1].unit_parameters[0] = 6; layers[1].unit_parameters[1] = 1;
        layers[2].type_layer = MYEA_LAYER_FULLY_CONNECTED; layers[2].unit_parameters[0] = 6;
        if (!nn.Compile(3, *T, MYEA_NETWORK_RECURRENT, layers)) return false;
        if (!nn.Set__Layer_Activation_Function(2, MYEA_AF_LINEAR) || !nn.Set__Layer_Normalization(1, MYEA_NORMALIZATION_BATCH_RENORMALIZATION)) return false;
        nn.Set__Loss_Function(MYEA_LOSS_MSE); nn.Set__Optimizer_Function(MYEA_OPTIMIZER_ADAM);
        nn.normalization_momentum_average = 0.5f; nn.batch_renormalization_r_correction_maximum = 2.f; nn.batch_renormalization_d_correction_maximum = 1.f;
    } else if (kind == "recurrent_residual") {
        // 6 -> IndRNN-8 tanh (BN before) -> residual block of 3 (block BN; members: IndRNN-8, IndRNN-8 with BN, LSTM 8 blocks of one cell)
        //   -> max pooling (kernel 2, stride 2, dilation 0) -> 4 linear, T = 3
        *T = 3; *n_in = 6; *n_out = 4;
        Layer_Parameters layers[8];
        layers[0].type_layer = MYEA_LAYER_FULLY_CONNECTED; layers[0].unit_parameters[0] = 6;
        layers[1].type_layer = MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT; layers[1].unit_parameters[0] = 8;
        layers[2].type_layer = MYEA_LAYER_RESIDUAL; layers[2].unit_parameters[0] = 3;
        layers[3].type_layer = layers[4].type_layer = MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT; layers[3].unit_parameters[0] = layers[4].unit_parameters[0] = 8;
        layers[5].type_layer = MYEA_LAYER_LSTM; layers[5].unit_parameters[0] = 8; layers[5].unit_parameters[1] = 1;
        layers[6].type_layer = MYEA_LAYER_MAX_POOLING; layers[6].unit_parameters[0] = 2; layers[6].unit_parameters[1] = 2;
        layers[7].type_layer = MYEA_LAYER_FULLY_CONNECTED; layers[7].unit_parameters[0] = 8;   // >= the LSTM member's cells: its bias vectors reach into these slots
        if (!nn.Compile(8, *T, MYEA_NETWORK_RECURRENT, layers)) return false;
        *n_out = 8;
        if (!nn.Set__Layer_Activation_Function(1, MYEA_AF_TANH) || !nn.Set__Layer_Activation_Function(3, MYEA_AF_TANH) || !nn.Set__Layer_Activation_Function(4, MYEA_AF_ISRLU) ||
            !nn.Set__Layer_Activation_Function(7, MYEA_AF_LINEAR) || !nn.Set__Layer_Normalization(1, MYEA_NORMALIZATION_BATCH_NORMALIZATION) ||
            !nn.Set__Layer_Normalization(2, MYEA_NORMALIZATION_BATCH_NORMALIZATION) || !nn.Set__Layer_Normalization(4, MYEA_NORMALIZATION_BATCH_NORMALIZATION) ||
            !nn.Set__Layer_Normalization(6, MYEA_NORMALIZATION_BATCH_NORMALIZATION)) return false;   // on a pooling layer: taken, means nothing
        nn.Set__Loss_Function(MYEA_LOSS_MSE); nn.Set__Optimizer_Function(MYEA_OPTIMIZER_AMSGRAD);
    } else {   // 8 -> 12 tanh -> residual block of 2 (block BN, ShakeDrop; members 10 and 14: wider than the shortcut) -> 4 linear
        *T = 1; *n_in = 8; *n_out = 4;
        Layer_Parameters layers[6];
        for (auto &l : layers) l.type_layer = MYEA_LAYER_FULLY_CONNECTED;
        layers[2].type_layer = MYEA_LAYER_RESIDUAL; layers[2].unit_parameters[0] = 2;
        layers[0].unit_parameters[0] = 8; layers[1].unit_parameters[0] = 12; layers[3].unit_parameters[0] = 10; layers[4].unit_parameters[0] = 14; layers[5].unit_parameters[0] = 4;
        if (!nn.Compile(6, *T, MYEA_NETWORK_FEEDFORWARD, layers)) return false;
        T_ shake[2] = {0.3f, 0.f}, keep[2] = {0.8f, 0.f};
        if (!nn.Set__Layer_Activation_Function(1, MYEA_AF_TANH) || !nn.Set__Layer_Activation_Function(3, MYEA_AF_RELU) || !nn.Set__Layer_Activation_Function(4, MYEA_AF_LEAKY_RELU) ||
            !nn.Set__Layer_Activation_Function(5, MYEA_AF_LINEAR) || !nn.Set__Layer_Normalization(2, MYEA_NORMALIZATION_BATCH_NORMALIZATION) ||
            !nn.Set__Layer_Normalization(4, MYEA_NORMALIZATION_BATCH_NORMALIZATION) || !nn.Set__Dropout(2, MYEA_DROPOUT_SHAKEDROP, shake) ||
            !nn.Set__Dropout(4, MYEA_DROPOUT_BERNOULLI_INVERTED, keep)) return false;
        nn.Set__Loss_Function(MYEA_LOSS_MSE); nn.Set__Optimizer_Function(MYEA_OPTIMIZER_ADAM);
    }
    for (size_t i = 0; i < nn.total_weights + nn.total_bias; ++i) nn.ptr_array_parameters[i] = rnd();
    for (size_t i = nn.total_weights + nn.total_bias; i < nn.total_parameters; ++i) nn.ptr_array_parameters[i] = 1.f + 0.5f * rnd();
    nn.loss_training = 0.125f; nn.loss_validating = 0.25f; nn.loss_testing = 0.5f;
    nn.accuracy_training = 75.f; nn.accuracy_validating = 62.5f; nn.accuracy_testing = 50.f; nn.accuracy_variance = 0.3f; nn.bit_fail_limit = 0.2f;
    return true;
}

int main(int argc, char **argv)
{
    if (argc < 3) return 2;
    const std::string dir = argv[1], kind = argv[2];
    const bool device = argc > 3;
    const size_t B = 7;
    size_t T, n_in, n_out;
    Neural_Network_HIP a, b;
    if (!build(a, kind, B, &T, &n_in, &n_out)) { std::printf("build failed\n"); return 1; }
    std::vector<float> x(B * T * n_in), y(B * T * n_out);
    for (float &v : x) v = 2.f * rnd();
    for (float &v : y) v = rnd();
    std::vector<const float *> xr(B), yr(B);
    for (size_t i = 0; i < B; ++i) { xr[i] = x.data() + i * T * n_in; yr[i] = y.data() + i * T * n_out; }
    if (device) {
        if (!a.Set__HIP(true)) return 1;
        a.type_state_propagation = MYEA_STATE_TRAINING;
        a.Clear_Training_Arrays();
        for (int s = 0; s < 2; ++s) {
            a.Forward_Pass(B, xr.data()); a.Compute__Error(B, yr.data()); a.Backward_Pass(B); a.Update_Derivative_Weight(B); a.Update_Parameter(B, B);
        }
    }
    if (!a.Save_Dimension_Parameters(dir + "/a.net") || !a.Save_General_Parameters(dir + "/a.nn")) { std::printf("save failed\n"); return 1; }
    if (!b.Load(dir + "/a.net", dir + "/a.nn")) { std::printf("load failed\n"); return 1; }
    if (!b.Update__Batch_Size(B)) return 1;
    if (device && !b.Set__HIP(true)) return 1;
    if (!b.Save_Dimension_Parameters(dir + "/b.net") || !b.Save_General_Parameters(dir + "/b.nn")) { std::printf("second save failed\n"); return 1; }
    if (slurp(dir + "/a.net") != slurp(dir + "/b.net") || slurp(dir + "/a.net").empty()) { std::printf("dimension files differ\n"); return 1; }
    if (slurp(dir + "/a.nn") != slurp(dir + "/b.nn") || slurp(dir + "/a.nn").empty()) { std::printf("general files differ\n"); return 1; }
    if (a.total_parameters != b.total_parameters) { std::printf("parameter counts differ\n"); return 1; }
    // every entry a kernel reads came back; an LSTM layer's first cell-count bias slots are not in the file (Prepare__Bias__LSTM
    // leaves [first, last) on the gate biases) and nothing reads them
    size_t differing = 0;
    for (size_t i = 0; i < a.total_parameters; ++i) differing += a.ptr_array_parameters[i] != b.ptr_array_parameters[i];
    std::printf("parameters %zu differing %zu\n", a.total_parameters, differing);
    {
        std::ofstream f(dir + "/params.bin", std::ios::binary);
        f.write(reinterpret_cast<const char *>(a.ptr_array_parameters), (std::streamsize)(a.total_parameters * sizeof(float)));
    }
    if (device) {
        a.type_state_propagation = b.type_state_propagation = MYEA_STATE_INFERENCE;
        a.Forward_Pass(B, xr.data()); b.Forward_Pass(B, xr.data());
        const myea_net_desc &d = a.Get__Descriptor();
        std::vector<float> ya(T * B * n_out), yb(T * B * n_out);
        if (myea_hip_download_tensor(a.Get__Device_Handle(), d.n_layers - 1, MYEA_TENSOR_OUTPUTS, ya.data(), ya.size()) != MYEA_OK ||
            myea_hip_download_tensor(b.Get__Device_Handle(), d.n_layers - 1, MYEA_TENSOR_OUTPUTS, yb.data(), yb.size()) != MYEA_OK) return 1;
        size_t bad = 0; double sum = 0;
        for (size_t i = 0; i < ya.size(); ++i) { bad += ya[i] != yb[i]; sum += std::fabs(ya[i]); }
        std::printf("inference outputs %zu differing %zu magnitude %.6g\n", ya.size(), bad, sum);
        if (bad || !(sum > 0)) return 1;
    }
    std::printf("OK\n");
    return 0;
}
