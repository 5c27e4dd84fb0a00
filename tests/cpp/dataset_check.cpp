// dataset_check.cpp — drives `Dataset_Mini_Batch_HIP` / `Dataset_HIP` (include/myea_dataset_hip.hpp) the way the reference's
// trainer drives `Dataset_Mini_Batch<T>::Training` and `Dataset<T>::Testing` (Neural_Network/Dataset__Mini_Batch.cpp:381-420,
// Neural_Network/Dataset.cpp:7758-7860): examples uploaded once, shuffled mini-batches gathered in HBM.
// usage: dataset_check <dir> <kind>   reads <dir>/{w,x,y}.bin; writes <dir>/params.bin and <dir>/order.bin (the shuffled index after
// every epoch, as float) and prints one line per epoch.  kind: "classify" (MLP, cross-entropy) or "regress" (LSTM, RMSE, R accuracy).
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "../../include/myea_dataset_hip.hpp"

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
    size_t N, T, n_in, n_out, bmax, per_batch, epochs = 2;
    Layer_Parameters layers[4];
    if (kind == "classify") {  // 11 -> 20 tanh -> 14 relu -> 5 softmax; momentum SGD, normalized weight decay
        N = 103; T = 1; n_in = 11; n_out = 5; bmax = 16; per_batch = 24;
        for (auto &l : layers) l.type_layer = MYEA_LAYER_FULLY_CONNECTED;
        layers[0].unit_parameters[0] = 11; layers[1].unit_parameters[0] = 20; layers[2].unit_parameters[0] = 14; layers[3].unit_parameters[0] = 5;
        if (!nn.Update__Batch_Size(bmax) || !nn.Compile(4, T, MYEA_NETWORK_FEEDFORWARD, layers)) return 1;
        if (!nn.Set__Layer_Activation_Function(1, MYEA_AF_TANH) || !nn.Set__Layer_Activation_Function(2, MYEA_AF_RELU) || !nn.Set__Layer_Activation_Function(3, MYEA_AF_SOFTMAX)) return 1;
        nn.Set__Loss_Function(MYEA_LOSS_CROSS_ENTROPY);
        nn.Set__Accuracy_Function(MYEA_ACCURACY_CROSS_ENTROPY);
        nn.Set__Optimizer_Function(MYEA_OPTIMIZER_GD);
        nn.learning_rate = 0.01f; nn.learning_momentum = 0.9f; nn.regularization__weight_decay = 0.02f;
    } else {  // 6 -> LSTM-9 -> LSTM-7 -> 7 linear over 5 steps, 1 delay; NosAdam; RMSE loss, R accuracy
        N = 60; T = 5; n_in = 6; n_out = 7; bmax = 8; per_batch = 20;
        layers[0].type_layer = MYEA_LAYER_FULLY_CONNECTED; layers[0].unit_parameters[0] = 6;
        layers[1].type_layer = MYEA_LAYER_LSTM; layers[1].unit_parameters[0] = 9; layers[1].unit_parameters[1] = 1;
        layers[2].type_layer = MYEA_LAYER_LSTM; layers[2].unit_parameters[0] = 7; layers[2].unit_parameters[1] = 1;
        layers[3].type_layer = MYEA_LAYER_FULLY_CONNECTED; layers[3].unit_parameters[0] = 7;
        if (!nn.Update__Batch_Size(bmax) || !nn.Compile(4, T, MYEA_NETWORK_RECURRENT, layers)) return 1;
        if (!nn.Set__Layer_Activation_Function(3, MYEA_AF_LINEAR)) return 1;
        nn.Set__Loss_Function(MYEA_LOSS_RMSE);
        nn.Set__Accuracy_Function(MYEA_ACCURACY_R);
        nn.Set__Optimizer_Function(MYEA_OPTIMIZER_NOSADAM);
        nn.number_time_delays = 1;
    }
    std::vector<float> w = read_f32(dir + "/w.bin"), x = read_f32(dir + "/x.bin"), y = read_f32(dir + "/y.bin");
    if (w.size() != nn.total_parameters || x.size() != N * T * n_in || y.size() != N * T * n_out) { std::printf("size mismatch\n"); return 1; }
    for (size_t i = 0; i < w.size(); ++i) nn.ptr_array_parameters[i] = w[i];
    if (!nn.Set__HIP(true)) return 1;
    nn.Clear_Training_Arrays();
    std::vector<const float *> xr(N), yr(N);
    for (size_t e = 0; e < N; ++e) { xr[e] = x.data() + e * T * n_in; yr[e] = y.data() + e * T * n_out; }
    Dataset_Mini_Batch_HIP data;
    if (!data.Allocate(N, n_in, n_out, T, xr.data(), yr.data()) || !data.Initialize(true, per_batch, 0, 12345ull)) return 1;
    std::printf("mini-batches %zu of %zu last %zu\n", data.Get__Number_Batch(), data.Get__Number_Examples_Per_Batch(), data.Get__Number_Examples_Last_Batch());
    std::vector<float> order;
    for (size_t e = 0; e < epochs; ++e) {
        const float loss = data.Training(&nn);
        std::printf("epoch %zu training loss %.9g accuracy %.9g\n", e, (double)loss, (double)nn.Get__Accuracy(Neural_Network_HIP::TYPE_DATASET_TRAINING));
        for (unsigned long long i : data.Get__Stochastic_Index()) order.push_back((float)i);
    }
    const float test_loss = data.Testing(&nn);
    std::printf("testing loss %.9g accuracy %.9g\n", (double)test_loss, (double)nn.Get__Accuracy(Neural_Network_HIP::TYPE_DATASET_TESTING));
    std::printf("time step %.1f epoch %.1f\n", (double)nn.optimizer_time_step, (double)nn.epoch_time_step);
    if (!nn.Copy__Parameters__Device_To_Host()) return 1;
    write_f32(dir + "/params.bin", nn.ptr_array_parameters, nn.total_parameters);
    write_f32(dir + "/order.bin", order.data(), order.size());
    // error behaviour: a dataset of another shape prints and returns the largest float
    Dataset_HIP other;
    std::vector<const float *> one(1, x.data());
    if (!other.Allocate(1, n_in + 1, n_out, T, one.data(), one.data())) return 1;
    std::printf("mismatch returns max: %d\n", other.Testing(&nn) == FLT_MAX ? 1 : 0);
    return 0;
}
