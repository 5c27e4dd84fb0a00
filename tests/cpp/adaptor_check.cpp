// adaptor_check.cpp — drives the C++ adaptor `Neural_Network_HIP` exactly as a host program drives the reference's
// `Neural_Network` (Compile -> Set__* -> Set__HIP -> the 4-call step loop + Update_Parameter, cf.
// Neural_Network_Launcher_Windows/Source_Files/debug.cpp:481-1555 and Neural_Network/Dataset.cpp:645-658).
// usage: adaptor_check <dir> <kind>   reads <dir>/{w,x,y,mask}.bin, writes <dir>/{params,grad}.bin and prints the loss.
//        adaptor_check <dir> dropout  host only: Dropout_Bernoulli's draws against the same draws made here.
// The step loop runs inside `#pragma omp parallel`, every thread of the team calling the step members, as the reference's
// Dataset::Train_Batch_BP does (Dataset.cpp:645-658); built with -fopenmp.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <string>
#include <vector>

#include "../../include/myea_nn_hip.hpp"

using namespace MyEA_HIP;

static std::vector<float> read_f32(const std::string &path)
{
    FILE *f = std::fopen(path.c_str(), "rb");
    if (!f) { std::printf("can not open %s\n", path.c_str()); std::exit(2); }
    std::fseek(f, 0, SEEK_END);
    long n = std::ftell(f);
    std::fseek(f, 0, SEEK_SET);
    std::vector<float> v(n / 4);
    if (std::fread(v.data(), 4, v.size(), f) != v.size()) std::exit(2);
    std::fclose(f);
    return v;
}
static void write_f32(const std::string &path, const float *p, size_t n)
{
    FILE *f = std::fopen(path.c_str(), "wb");
    std::fwrite(p, 4, n, f);
    std::fclose(f);
}

int main(int argc, char **argv)
{
    if (argc < 3) return 2;
    const std::string dir = argv[1], kind = argv[2];
    Neural_Network_HIP nn;
    size_t B, T, n_in, n_out, steps = 3;
    if (kind == "dropout") {
        // FC 10 (Bernoulli .8 on the inputs) -> 12 (Bernoulli .6) -> 9 (inverted .5) -> 7 (Bernoulli, retention 0) -> 4, T = 3
        Layer_Parameters layers[5];
        for (auto &l : layers) l.type_layer = MYEA_LAYER_FULLY_CONNECTED;
        const size_t units[5] = {10, 12, 9, 7, 4};
        for (int i = 0; i < 5; ++i) layers[i].unit_parameters[0] = units[i];
        T = 3;
        if (!nn.Update__Batch_Size(2) || !nn.Compile(5, T, MYEA_NETWORK_RECURRENT, layers)) return 1;
        T_ k0[2] = {0.8f, 0.f}, k1[2] = {0.6f, 0.f}, k2[2] = {0.5f, 0.f}, k3[2] = {0.f, 0.f};
        if (!nn.Set__Dropout(0, MYEA_DROPOUT_BERNOULLI, k0) || !nn.Set__Dropout(1, MYEA_DROPOUT_BERNOULLI, k1) ||
            !nn.Set__Dropout(2, MYEA_DROPOUT_BERNOULLI_INVERTED, k2) || !nn.Set__Dropout(3, MYEA_DROPOUT_BERNOULLI, k3)) return 1;
        if (nn.total_layers != 5 || nn.ptr_last_layer != nn.ptr_array_layers + 5 || nn.ptr_array_layers[2].type_dropout != MYEA_DROPOUT_BERNOULLI_INVERTED) return 1;
        const size_t total = (10 + 12 + 9 + 7 + 4) * T;
        if (nn.Get__Descriptor().total_mask_units != total) { std::printf("mask units %llu\n", (unsigned long long)nn.Get__Descriptor().total_mask_units); return 1; }
        nn.Set__Seed__Dropout_Bernoulli(1234u);
        nn.Dropout_Bernoulli();
        // the same draws, made here: layer order, [time step][unit], the distribution re-parameterised when the probability changes
        std::mt19937 gen(1234u);
        std::bernoulli_distribution dist(0.5);
        std::vector<bool> want(total, true);
        dist.param(std::bernoulli_distribution::param_type(0.8f));
        for (size_t i = 0; i < 10 * T; ++i) want[i] = dist(gen);
        dist.param(std::bernoulli_distribution::param_type(0.6f));
        for (size_t i = 0; i < 12 * T; ++i) want[10 * T + i] = dist(gen);
        for (size_t i = 0; i < 7 * T; ++i) want[(10 + 12 + 9) * T + i] = false;     // retention 0: all dropped, no draw
        size_t kept0 = 0;
        for (size_t i = 0; i < total; ++i) {
            if (nn.ptr_array_units_mask_dropout_bernoulli[i] != want[i]) { std::printf("mask %zu differs\n", i); return 1; }
            if (i < 10 * T && want[i]) ++kept0;
        }
        if (kept0 == 0 || kept0 == 10 * T) return 1;
        std::printf("dropout ok\n");
        return 0;
    }
    if (kind == "mlp") {  // FC 20 -> 32 (BN before, ReLU, inverted dropout .5) -> 24 tanh -> 6 softmax, Nesterov
        B = 16; T = 1; n_in = 20; n_out = 6;
        Layer_Parameters layers[4];
        for (auto &l : layers) l.type_layer = MYEA_LAYER_FULLY_CONNECTED;
        layers[0].unit_parameters[0] = 20; layers[1].unit_parameters[0] = 32; layers[2].unit_parameters[0] = 24; layers[3].unit_parameters[0] = 6;
        if (!nn.Update__Batch_Size(B)) return 1;
        if (!nn.Compile(4, T, MYEA_NETWORK_FEEDFORWARD, layers)) return 1;
        T_ keep[2] = {0.5f, 0.f};
        if (!nn.Set__Layer_Activation_Function(1, MYEA_AF_RELU) || !nn.Set__Layer_Activation_Function(2, MYEA_AF_TANH) ||
            !nn.Set__Layer_Activation_Function(3, MYEA_AF_SOFTMAX) || !nn.Set__Layer_Normalization(1, MYEA_NORMALIZATION_BATCH_NORMALIZATION, true) ||
            !nn.Set__Dropout(1, MYEA_DROPOUT_BERNOULLI_INVERTED, keep)) return 1;
        nn.Set__Loss_Function(MYEA_LOSS_CROSS_ENTROPY);
        nn.Set__Accuracy_Function(MYEA_ACCURACY_CROSS_ENTROPY);
        nn.Set__Optimizer_Function(MYEA_OPTIMIZER_GD);
        nn.use_Nesterov = true;
    } else if (kind == "indrnn") {  // 8 -> IndRNN-16 (default: ReLU) -> IndRNN-12 tanh, clip [-0.5, 0.75] -> FC-4 linear, GD
        B = 6; T = 5; n_in = 8; n_out = 4;
        Layer_Parameters layers[4];
        for (auto &l : layers) l.type_layer = MYEA_LAYER_FULLY_CONNECTED;
        layers[1].type_layer = layers[2].type_layer = MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT;
        layers[0].unit_parameters[0] = 8; layers[1].unit_parameters[0] = 16; layers[2].unit_parameters[0] = 12; layers[3].unit_parameters[0] = 4;
        if (!nn.Update__Batch_Size(B)) return 1;
        if (!nn.Compile(4, T, MYEA_NETWORK_RECURRENT, layers)) return 1;
        // Compile's default bounds: +-2^(1/T) for the rectifier; a layer on its default follows the activation and the clip value
        if (!nn.Check__Use__Regularization__Constraint_Recurrent_Weight__Default(1) || nn.Check__Use__Regularization__Constraint_Recurrent_Weight__Default(3)) return 1;
        if (std::fabs(nn.Get__Descriptor().layers[1].constraint_recurrent_weight_upper_bound - std::pow(2.f, 1.f / 5.f)) > 1e-6f) return 1;
        if (!nn.Set__Layer_Activation_Function(2, MYEA_AF_TANH) || !nn.Check__Use__Regularization__Constraint_Recurrent_Weight__Default(2)) return 1;
        if (std::fabs(nn.Get__Descriptor().layers[2].constraint_recurrent_weight_upper_bound - std::pow(2.f / std::pow(0.9f, 0.5f), 1.f / 5.f)) > 1e-6f) return 1;
        if (!nn.Set__Clip_Gradient(3.0f)) return 1;
        if (std::fabs(nn.Get__Descriptor().layers[1].constraint_recurrent_weight_upper_bound - std::pow(3.f, 1.f / 5.f)) > 1e-6f) return 1;
        if (!nn.Set__Regularization__Constraint_Recurrent_Weight(2, -0.5f, 0.75f) || nn.Set__Regularization__Constraint_Recurrent_Weight(3, -1.f, 1.f) ||
            nn.Set__Regularization__Constraint_Recurrent_Weight(2, 1.f, -1.f)) return 1;
        if (!nn.Set__Clip_Gradient(1.0f) || nn.Get__Descriptor().layers[2].constraint_recurrent_weight_upper_bound != 0.75f) return 1;
        if (!nn.Set__Layer_Activation_Function(3, MYEA_AF_LINEAR)) return 1;
        nn.Set__Loss_Function(MYEA_LOSS_MSE);
        nn.Set__Optimizer_Function(MYEA_OPTIMIZER_GD);
    } else if (kind == "example") {
        // The network of the reference's worked example, built with its sequence of calls (Neural_Network_Launcher_Windows/Source_Files/
        // debug.cpp:693-1075 the layer list, :1160-1230 time delays and activations, :1317 the constraint, :1503-1520 the normalisation of
        // EVERY hidden layer - residual and pooling layers included): sMNIST rows, an independently recurrent first hidden layer, three
        // groups of three residual blocks of three independently recurrent members, 9 units narrower in all over the nine blocks, a max
        // pooling (kernel 2, stride 2, dilation 0) between the groups, ISRLU, softmax head, AMSGrad, max-norm constraint 8
        B = 12; T = 5; n_in = 28; n_out = 10;
        std::vector<Layer_Parameters> lp;
        Layer_Parameters l;
        l.type_layer = MYEA_LAYER_FULLY_CONNECTED; l.unit_parameters[0] = 28; lp.push_back(l);
        l.type_layer = MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT; l.unit_parameters[0] = 32; lp.push_back(l);
        double width = 32.0;
        const double widening = -9.0 / 9.0;
        for (int group = 0; group < 3; ++group) {
            if (group) {
                l.type_layer = MYEA_LAYER_MAX_POOLING;
                l.unit_parameters[0] = 2; l.unit_parameters[1] = 2; l.unit_parameters[2] = 0; l.unit_parameters[3] = 0; l.unit_parameters[4] = 0;
                lp.push_back(l);
            }
            for (int block = 0; block < 3; ++block) {
                l.type_layer = MYEA_LAYER_RESIDUAL; l.unit_parameters[0] = 3; lp.push_back(l);
                width += widening;
                l.type_layer = MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT; l.unit_parameters[0] = (size_t)width;
                for (int member = 0; member < 3; ++member) lp.push_back(l);
            }
        }
        l.type_layer = MYEA_LAYER_FULLY_CONNECTED; l.unit_parameters[0] = 10; lp.push_back(l);
        if (!nn.Update__Batch_Size(B)) return 1;
        if (!nn.Compile(lp.size(), T, MYEA_NETWORK_FEEDFORWARD, lp.data())) return 1;
        if (!nn.Set__Number_Time_Delays(T - 1)) return 1;
        for (size_t i = 0; i < lp.size(); ++i) if (!nn.Set__Layer_Activation_Steepness(i, 1.f)) return 1;
        for (size_t i = 1; i + 1 < lp.size(); ++i) if (!nn.Set__Layer_Activation_Function(i, MYEA_AF_ISRLU)) return 1;
        if (!nn.Set__Layer_Activation_Function(lp.size() - 1, MYEA_AF_SOFTMAX)) return 1;
        nn.Set__Loss_Function(MYEA_LOSS_CROSS_ENTROPY);
        nn.Set__Accuracy_Function(MYEA_ACCURACY_CROSS_ENTROPY);
        nn.Set__Optimizer_Function(MYEA_OPTIMIZER_AMSGRAD);
        if (!nn.Set__Regularization__Max_Norm_Constraints(8.f)) return 1;
        for (size_t i = 1; i + 1 < lp.size(); ++i) if (!nn.Set__Layer_Normalization(i, MYEA_NORMALIZATION_BATCH_NORMALIZATION, true)) return 1;
        if (!nn.Set__Normalization_Momentum_Average(1.f) || !nn.Set__Normalization_Epsilon(0.1f)) return 1;
    } else {  // LSTM 8 -> 2 x LSTM-12 -> FC-12 linear, AMSGrad, clip 1.0
        B = 6; T = 5; n_in = 8; n_out = 12;
        Layer_Parameters layers[4];
        layers[0].type_layer = MYEA_LAYER_FULLY_CONNECTED; layers[0].unit_parameters[0] = 8;
        layers[1].type_layer = MYEA_LAYER_LSTM; layers[1].unit_parameters[0] = 12; layers[1].unit_parameters[1] = 1;
        layers[2].type_layer = MYEA_LAYER_LSTM; layers[2].unit_parameters[0] = 6; layers[2].unit_parameters[1] = 2;
        layers[3].type_layer = MYEA_LAYER_FULLY_CONNECTED; layers[3].unit_parameters[0] = 12;
        if (!nn.Update__Batch_Size(B)) return 1;
        if (!nn.Compile(4, T, MYEA_NETWORK_RECURRENT, layers)) return 1;
        if (!nn.Set__Layer_Activation_Function(3, MYEA_AF_LINEAR)) return 1;
        nn.Set__Loss_Function(MYEA_LOSS_MSE);
        nn.Set__Optimizer_Function(MYEA_OPTIMIZER_AMSGRAD);
        nn.Set__Clip_Gradient(true);
        nn.Set__Clip_Gradient(1.0f);
    }
    std::vector<float> w = read_f32(dir + "/w.bin"), x = read_f32(dir + "/x.bin"), y = read_f32(dir + "/y.bin"), m = read_f32(dir + "/mask.bin");
    if (w.size() != nn.total_parameters) { std::printf("parameter count %zu != %zu\n", w.size(), nn.total_parameters); return 1; }
    for (size_t i = 0; i < w.size(); ++i) nn.ptr_array_parameters[i] = w[i];
    for (size_t i = 0; i < m.size() && i < nn.Get__Descriptor().total_mask_units; ++i) nn.ptr_array_units_mask_dropout_bernoulli[i] = m[i] != 0.f;
    if (!nn.Set__HIP(true)) return 1;
    nn.type_state_propagation = MYEA_STATE_TRAINING;
    nn.Clear_Training_Arrays();
    std::vector<const float *> xr(B), yr(B);
    for (size_t b = 0; b < B; ++b) { xr[b] = x.data() + b * T * n_in; yr[b] = y.data() + b * T * n_out; }
    std::vector<float> grad(nn.total_parameters);
    int failed = 0;
    // every thread of the team walks the loop and makes the calls; the class lets one of them through
#pragma omp parallel num_threads(3)
    for (size_t s = 0; s < steps; ++s) {
#pragma omp barrier
#pragma omp master
        nn.Reset__Loss();
        nn.Forward_Pass(B, xr.data());
        nn.Compute__Error(B, yr.data());
        nn.Backward_Pass(B);
        nn.Update_Derivative_Weight(B, nn.ptr_array_layers + 1, nn.ptr_last_layer);
#pragma omp barrier
#pragma omp master
        {
            if (s + 1 == steps && !nn.Copy__Derivatives_Parameters__Device_To_Host(grad.data())) failed = 1;
            std::printf("step %zu loss %.9g\n", s, (double)nn.Get__Loss());
        }
        nn.Update_Parameter(B, B);
    }
    if (failed) return 1;
    if (!nn.Copy__Parameters__Device_To_Host()) return 1;
    write_f32(dir + "/params.bin", nn.ptr_array_parameters, nn.total_parameters);
    write_f32(dir + "/grad.bin", grad.data(), grad.size());
    // error behaviour: a batch larger than the allocated one prints and returns, leaving the network usable
    std::vector<const float *> big(B + 1, x.data());
    nn.Forward_Pass(B + 1, big.data());
    std::printf("time step %.1f\n", (double)nn.optimizer_time_step);
    return 0;
}
