// myea_nn_hip.hpp — header-only C++ host adaptor over the C ABI of include/myea_hip.h.
//
// `Neural_Network_HIP` mirrors the part of the reference's `class Neural_Network`
// (Header_Files/Neural_Network/Data.hpp:760-3294) that sits on the training hot path: same method names, same
// argument meaning (batch_size_received, arrays of per-example row pointers, layer indices), same error behaviour
// (`bool` setters that print and return false; `void` step functions that print and return), same public training
// fields.  A host program written against the reference (see Neural_Network_Launcher_Windows/Source_Files/debug.cpp:
// 481-1555 for the call order) switches to the MI355X path by swapping the class.
//
// Everything here is host code; the device work happens behind myea_hip_*.
#pragma once

#include <cstdio>
#include <cfloat>
#include <cmath>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "myea_hip.h"

namespace MyEA_HIP {

typedef float T_;  // COMPILE_FLOAT (Common_Library/include/Configuration/DTypes.hpp:20-32)

// Header_Files/Neural_Network/Data.hpp:56-80
struct Layer_Parameters {
    bool use_bidirectional = false;
    unsigned int type_layer = MYEA_LAYER_NONE;  // MYEA_LAYER_*
    // [0] FC: neurons, LSTM: blocks, RESIDUAL: block depth.  [1] LSTM: cells per block.
    // pooling layers: [0] kernel size, [1] stride, [2] padding, [3] dilation, [4] ceil mode.
    size_t unit_parameters[5u] = {0};
};

// The reference's callers hand `struct Layer` pointers to Update_Derivative_Weight (Dataset.cpp:655-657:
// ptr_array_layers + 1, ptr_last_layer).  Here a Layer is a read-only view of one descriptor entry; what matters to the
// step functions is its position in ptr_array_layers.
struct Layer {
    unsigned int type_layer = MYEA_LAYER_NONE, type_dropout = MYEA_DROPOUT_NONE;
    bool use_bidirectional = false;
    T_ dropout_values[3] = {0.f, 0.f, 0.f};
};

class Neural_Network_HIP {
public:
    // ---- public training fields, defaults of Data.hpp:2929-2970 ----
    T_ learning_rate = 0.01f, learning_rate_final = 0.1f, learning_momentum = 0.9f, learning_gamma = 1e-3f;
    T_ adam_learning_rate = 0.001f, adam_beta1 = 0.9f, adam_beta2 = 0.999f, adam_epsilon = 1e-8f;
    T_ regularization__weight_decay = 0.f, clip_gradient = 1.f, accuracy_variance = 0.49f, bit_fail_limit = 0.35f;
    T_ normalization_momentum_average = 0.999f, normalization_epsilon = 1e-5f;
    T_ batch_renormalization_r_correction_maximum = 1.f, batch_renormalization_d_correction_maximum = 0.f;
    bool use_Nesterov = false, use_adam_bias_correction = true, use_clip_gradient = false;
    bool use_normalized_weight_decay = true, use_Warm_Restarts = false;
    T_ adam_gamma = 0.1f, regularization__max_norm_constraints = 0.f;
    T_ rprop_increase_factor = 1.2f, rprop_decrease_factor = 0.5f, rprop_delta_min = 1e-6f, rprop_delta_max = 50.f, rprop_delta_zero = 0.1f;
    T_ warm_restarts_decay_learning_rate = 1.f, warm_restarts_minimum_learning_rate = 1e-7f, warm_restarts_multiplier = 2.f;
    // written by the caller's epoch loop and by the library (Clear_Optimizer, Warm_Restarts_Decay, the NosAdam step):
    // pushed before and read back after every call that may change them
    T_ optimizer_time_step = 0.f, epoch_time_step = 1.f, adam_previous_beta2 = 0.f;
    T_ loss_rprop = FLT_MAX, previous_loss_rprop = FLT_MAX;
    T_ warm_restarts_maximum_learning_rate = 1.f, warm_restarts_T_i = 1.f;
    // the values a warm-restart schedule starts from; these are what the checkpoint keeps (Neural_Network__Save.cpp:85-88)
    T_ warm_restarts_initial_maximum_learning_rate = 1.f, warm_restarts_initial_T_i = 1.f;
    unsigned int type_optimizer_function = MYEA_OPTIMIZER_NONE, type_loss_function = MYEA_LOSS_NONE;
    unsigned int type_accuracy_function = MYEA_ACCURACY_DISTANCE;
    unsigned int type_state_propagation = MYEA_STATE_INFERENCE;
    size_t number_time_delays = 0, number_recurrent_depth = 1, batch_size = 1;
    size_t total_parameters = 0, total_weights = 0, total_bias = 0;
    // public host copies, written by the caller like the reference's members and pushed with the Copy__* calls
    T_ *ptr_array_parameters = nullptr;                      // [total_parameters]
    bool *ptr_array_units_mask_dropout_bernoulli = nullptr;  // [(sum of AF units) * T], all true after Compile
    struct Layer *ptr_array_layers = nullptr;                // [total_layers], refreshed by Compile and the Set__* calls
    struct Layer const *ptr_last_layer = nullptr;            // ptr_array_layers + total_layers
    size_t total_layers = 0;

    Neural_Network_HIP() { std::memset(&desc_, 0, sizeof(desc_)); }
    ~Neural_Network_HIP() { Deallocate(); }
    Neural_Network_HIP(const Neural_Network_HIP &) = delete;
    Neural_Network_HIP &operator=(const Neural_Network_HIP &) = delete;

    // Neural_Network::Compile (Data.hpp:2531; Neural_Network__Compile.cpp:426).  maximum_allowable_memory is accepted
    // for signature compatibility; device memory is sized from the descriptor.
    bool Compile(size_t number_layers, size_t number_recurrent_depth_received, unsigned int type_network,
                 Layer_Parameters const *ptr_array_layers, size_t maximum_allowable_memory = 0)
    {
        (void)maximum_allowable_memory;
        if (number_layers < 2 || number_layers > MYEA_MAX_LAYERS || ptr_array_layers == nullptr) return Fail("Compile", "bad layer count");
        if (number_recurrent_depth_received == 0) return Fail("Compile", "recurrent depth can not be zero");
        Deallocate();
        std::memset(&desc_, 0, sizeof(desc_));
        desc_.type_network = type_network;
        desc_.n_layers = (uint32_t)number_layers;
        desc_.number_recurrent_depth = (uint32_t)number_recurrent_depth_received;
        desc_.batch_size = (uint32_t)batch_size;
        number_recurrent_depth = number_recurrent_depth_received;
        for (size_t i = 0; i < number_layers; ++i) {
            myea_layer_desc &l = desc_.layers[i];
            l.type_layer = ptr_array_layers[i].type_layer;
            l.use_bidirectional = ptr_array_layers[i].use_bidirectional;
            l.n_units = (uint32_t)ptr_array_layers[i].unit_parameters[0];
            l.n_cells_per_block = l.type_layer == MYEA_LAYER_LSTM ? (uint32_t)ptr_array_layers[i].unit_parameters[1] : 0;
            if (l.type_layer == MYEA_LAYER_RESIDUAL) { l.block_depth = l.n_units; l.n_units = 0; }
            if (l.type_layer == MYEA_LAYER_AVERAGE_POOLING || l.type_layer == MYEA_LAYER_MAX_POOLING) {
                // kernel size, stride, padding, dilation, ceil mode (Assign__Layer, Neural_Network__Compile.cpp:51-58); the width follows
                for (int k = 0; k < 5; ++k) l.pooling_values[k] = (uint32_t)ptr_array_layers[i].unit_parameters[k];
                l.n_units = 0;
            }
            // Compile's defaults: FC layers start as sigmoid with steepness 1 (Neural_Network__Compile.cpp:572-590),
            // independently recurrent layers as rectifiers with the default clip of their self weights (:593-627)
            l.type_activation_function = (i > 0 && l.type_layer == MYEA_LAYER_FULLY_CONNECTED) ? MYEA_AF_SIGMOID : MYEA_AF_NONE;
            if (l.type_layer == MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT) {
                l.type_activation_function = MYEA_AF_RELU;
                Compute__Regularization__Constraint_Recurrent_Weight__Default(i, &l.constraint_recurrent_weight_lower_bound, &l.constraint_recurrent_weight_upper_bound);
            }
            l.activation_steepness = 1.f;
            l.use_layer_normalization_before_activation = 1;
            l.dropout_values[0] = 1.f;
            l.alpha_sparsity = 1.f;   // Data.hpp:734
        }
        return Relayout("Compile");
    }

    bool Set__Layer_Activation_Function(size_t index_layer, unsigned int type_activation_function)
    {
        if (!CheckLayer("Set__Layer_Activation_Function", index_layer)) return false;
        if (type_activation_function == MYEA_AF_NONE || type_activation_function >= MYEA_AF_LENGTH) return Fail("Set__Layer_Activation_Function", "activation function out of range");
        // a layer still on the default clip of its self weights follows the new activation's default (Train.cpp:538-640)
        const bool follows = Check__Use__Regularization__Constraint_Recurrent_Weight__Default(index_layer);
        desc_.layers[index_layer].type_activation_function = type_activation_function;
        if (follows) Set__Regularization__Constraint_Recurrent_Weight__Default(index_layer);
        return Dirty();
    }
    // Compute__Regularization__Constraint_Recurrent_Weight__Default
    // (Neural_Network__Regularization__Constraint_Recurrent_Weight.cpp:33-75): +-MAG^(1/T) with MAG = clip_gradient kept in
    // [2, 10]; for the symmetric activations MAG is first divided by 0.9^(T/10)
    void Compute__Regularization__Constraint_Recurrent_Weight__Default(size_t index_layer, T_ *lower_bound, T_ *upper_bound) const
    {
        const T_ MAG = clip_gradient < 2.f ? 2.f : (clip_gradient > 10.f ? 10.f : clip_gradient), T = (T_)number_recurrent_depth;
        T_ bound;
        switch (desc_.layers[index_layer].type_activation_function) {
        case MYEA_AF_COSINE_SYMMETRIC: case MYEA_AF_ELLIOT_SYMMETRIC: case MYEA_AF_GAUSSIAN_SYMMETRIC: case MYEA_AF_LINEAR_PIECE_SYMMETRIC:
        case MYEA_AF_SINE_SYMMETRIC: case MYEA_AF_TANH: case MYEA_AF_TANH_STEPWISE: case MYEA_AF_THRESHOLD_SYMMETRIC:
            bound = std::pow(MAG / std::pow(0.9f, T / 10.f), 1.f / T);
            break;
        default: bound = std::pow(MAG, 1.f / T); break;
        }
        *lower_bound = -bound; *upper_bound = bound;
    }
    bool Check__Use__Regularization__Constraint_Recurrent_Weight__Default(size_t index_layer) const
    {
        if (index_layer >= desc_.n_layers || desc_.layers[index_layer].type_layer != MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT) return false;
        T_ lo, hi;
        Compute__Regularization__Constraint_Recurrent_Weight__Default(index_layer, &lo, &hi);
        const myea_layer_desc &l = desc_.layers[index_layer];
        return std::fabs(l.constraint_recurrent_weight_lower_bound - lo) <= 1e-8 && std::fabs(l.constraint_recurrent_weight_upper_bound - hi) <= 1e-8;
    }
    // Set__Regularization__Constraint_Recurrent_Weight (:143-229): recurrent hidden layers only, lower <= upper
    bool Set__Regularization__Constraint_Recurrent_Weight(size_t index_layer, T_ lower_bound, T_ upper_bound)
    {
        if (!CheckLayer("Set__Regularization__Constraint_Recurrent_Weight", index_layer)) return false;
        if (index_layer + 1 == desc_.n_layers) return Fail("Set__Regularization__Constraint_Recurrent_Weight", "layer received as argument is the output layer");
        if (desc_.layers[index_layer].type_layer != MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT) return Fail("Set__Regularization__Constraint_Recurrent_Weight", "can not constrain the recurrent weight of this type of layer");
        if (lower_bound > upper_bound) return Fail("Set__Regularization__Constraint_Recurrent_Weight", "lower bound greater than upper bound");
        desc_.layers[index_layer].constraint_recurrent_weight_lower_bound = lower_bound;
        desc_.layers[index_layer].constraint_recurrent_weight_upper_bound = upper_bound;
        return Dirty();
    }
    bool Set__Regularization__Constraint_Recurrent_Weight__Default(size_t index_layer)
    {
        if (!CheckLayer("Set__Regularization__Constraint_Recurrent_Weight__Default", index_layer)) return false;
        T_ lo, hi;
        Compute__Regularization__Constraint_Recurrent_Weight__Default(index_layer, &lo, &hi);
        return Set__Regularization__Constraint_Recurrent_Weight(index_layer, lo, hi);
    }
    // Train.cpp:676-720: a steepness in [0, 1], any layer of the network (the example program walks all of them, the input layer,
    // residual and pooling layers included: those have no activation to steepen and the value means nothing there)
    bool Set__Layer_Activation_Steepness(size_t index_layer, T_ activation_steepness)
    {
        if (activation_steepness < 0.f || activation_steepness > 1.f) return Fail("Set__Layer_Activation_Steepness", "activation steepness outside [0, 1]");
        if (index_layer >= desc_.n_layers) return Fail("Set__Layer_Activation_Steepness", "layer index overflow");
        desc_.layers[index_layer].activation_steepness = activation_steepness;
        return Dirty();
    }
    // Data.hpp:2697; `use_layer_normalization_before_activation` is a public Layer field in the reference
    bool Set__Layer_Normalization(size_t index_layer, unsigned int type_layer_normalization, bool use_layer_normalization_before_activation = true)
    {
        if (!CheckLayer("Set__Layer_Normalization", index_layer)) return false;
        desc_.layers[index_layer].type_normalization = type_layer_normalization;
        desc_.layers[index_layer].use_layer_normalization_before_activation = use_layer_normalization_before_activation;
        return Relayout("Set__Layer_Normalization");
    }
    // Data.hpp:2667; value_dropout[0] = retention probability
    bool Set__Dropout(size_t index_layer, unsigned int type_layer_dropout, T_ const value_dropout[], bool scale_weights = true)
    {
        (void)scale_weights;
        if (index_layer >= desc_.n_layers) return Fail("Set__Dropout", "layer index overflow");
        if (value_dropout == nullptr || value_dropout[0] < 0.f || value_dropout[0] > 1.f) return Fail("Set__Dropout", "retention probability out of [0, 1]");
        desc_.layers[index_layer].type_dropout = type_layer_dropout;
        desc_.layers[index_layer].dropout_values[0] = value_dropout[0];
        // Set__Dropout_Gaussian keeps p / (1 - p), the spread of the multiplicative noise (Neural_Network__Dropout.cpp:509-565)
        if (type_layer_dropout == MYEA_DROPOUT_GAUSSIAN)
            desc_.layers[index_layer].dropout_values[0] = value_dropout[0] == 1.f ? 0.f : (T_)((double)value_dropout[0] / (1.0 - (double)value_dropout[0]));
        if (type_layer_dropout == MYEA_DROPOUT_ZONEOUT) desc_.layers[index_layer].dropout_values[1] = value_dropout[1];   // cell-output probability
        return Dirty();
    }
    // Set__K_Sparsity / Set__Alpha_Sparsity (Neural_Network__K_Sparse.cpp:21-190): hidden layers; size_t(k * alpha) may not
    // exceed the layer's width
    bool Set__K_Sparsity(size_t index_layer, size_t k_sparsity)
    {
        if (!CheckLayer("Set__K_Sparsity", index_layer)) return false;
        if (index_layer + 1 == desc_.n_layers) return Fail("Set__K_Sparsity", "layer received as argument is the output layer");
        myea_layer_desc &l = desc_.layers[index_layer];
        if (l.k_sparsity == k_sparsity) return true;
        if ((size_t)((T_)k_sparsity * l.alpha_sparsity) > (size_t)myea_net_desc_number_outputs(&desc_, (uint32_t)index_layer)) return Fail("Set__K_Sparsity", "k-sparse can not be greater than the number of outputs");
        l.k_sparsity = (uint32_t)k_sparsity;
        return Dirty();
    }
    bool Set__Alpha_Sparsity(size_t index_layer, T_ alpha_sparsity)
    {
        if (!CheckLayer("Set__Alpha_Sparsity", index_layer)) return false;
        if (index_layer + 1 == desc_.n_layers) return Fail("Set__Alpha_Sparsity", "layer received as argument is the output layer");
        if (alpha_sparsity < 0.f) return Fail("Set__Alpha_Sparsity", "alpha k-sparse can not be less than zero");
        myea_layer_desc &l = desc_.layers[index_layer];
        if ((size_t)((T_)l.k_sparsity * alpha_sparsity) > (size_t)myea_net_desc_number_outputs(&desc_, (uint32_t)index_layer)) return Fail("Set__Alpha_Sparsity", "k-sparse can not be greater than the number of outputs");
        l.alpha_sparsity = alpha_sparsity;
        return Dirty();
    }
    void Set__Loss_Function(unsigned int f) { type_loss_function = f; }
    void Set__Accuracy_Function(unsigned int f) { type_accuracy_function = f; }
    void Set__Optimizer_Function(unsigned int f) { type_optimizer_function = f; }
    void Set__Clip_Gradient(bool use) { use_clip_gradient = use; }
    // Set__Clip_Gradient (Neural_Network__Clip_Gradient.cpp:20-80): layers on the default clip of their self weights follow
    bool Set__Clip_Gradient(T_ value)
    {
        bool follows[MYEA_MAX_LAYERS];
        for (size_t i = 0; i < desc_.n_layers; ++i) follows[i] = Check__Use__Regularization__Constraint_Recurrent_Weight__Default(i);
        clip_gradient = value;
        for (size_t i = 0; i < desc_.n_layers; ++i)
            if (follows[i] && !Set__Regularization__Constraint_Recurrent_Weight__Default(i)) return false;
        return true;
    }
    // Neural_Network__Regularization__Max_Norm_Constraints.cpp:24-46: a negative bound prints and returns false
    bool Set__Regularization__Max_Norm_Constraints(T_ v)
    {
        if (v < 0.f) return Fail("Set__Regularization__Max_Norm_Constraints", "max-norm constraints less than zero");
        regularization__max_norm_constraints = v;
        return true;
    }
    bool Set__Accurancy_Variance(T_ v) { accuracy_variance = v; return true; }
    bool Set__Number_Time_Delays(size_t n) { if (n > number_recurrent_depth) return Fail("Set__Number_Time_Delays", "time delays exceed the recurrent depth"); number_time_delays = n; return true; }
    bool Set__Normalization_Momentum_Average(T_ v) { normalization_momentum_average = v; return true; }
    bool Set__Normalization_Epsilon(T_ v) { normalization_epsilon = v; return true; }
    bool Set__Batch_Renormalization_r_Correction_Maximum(T_ v) { batch_renormalization_r_correction_maximum = v; return true; }
    bool Set__Batch_Renormalization_d_Correction_Maximum(T_ v) { batch_renormalization_d_correction_maximum = v; return true; }

    // Data.hpp:2559
    bool Update__Batch_Size(size_t desired_batch_size, bool force_update = false)
    {
        (void)force_update;
        if (desired_batch_size == 0) return Fail("Update__Batch_Size", "batch size can not be zero");
        batch_size = desired_batch_size;
        desc_.batch_size = (uint32_t)desired_batch_size;
        return Dirty();
    }

    // The seam where the reference has Set__CUDA (Data.hpp:3116): creates the device object from the current
    // descriptor and uploads parameters and masks.
    bool Set__HIP(bool use_hip)
    {
        pushed_valid_ = false;
        if (!use_hip) { if (net_) { myea_hip_destroy(net_); net_ = nullptr; } return true; }
        if (net_) { myea_hip_destroy(net_); net_ = nullptr; }
        if (myea_hip_create(&desc_, &net_) != MYEA_OK) return Fail("Set__HIP", myea_hip_last_error());
        // running statistics a checkpoint brought along (Load)
        for (size_t li = 0; li < norm_means_averages_.size() && li < desc_.n_layers; ++li) {
            if (norm_means_averages_[li].empty()) continue;
            if (desc_.layers[li].type_layer == MYEA_LAYER_LSTM) {   // held as [direction][group][T][K], uploaded group by group
                const size_t per = (size_t)desc_.number_recurrent_depth * desc_.layers[li].n_units;
                for (size_t dg = 0; dg * per < norm_means_averages_[li].size(); ++dg) {
                    const int sel = MYEA_TENSOR_LSTM_NORM_GROUP((int)(dg % 9)) | (dg >= 9 ? MYEA_TENSOR_DIRECTION_BACKWARD : 0);
                    if (!Ok("Set__HIP", myea_hip_upload_tensor(net_, li, MYEA_TENSOR_NORM_MEANS_AVERAGES | sel, norm_means_averages_[li].data() + dg * per, per)) ||
                        !Ok("Set__HIP", myea_hip_upload_tensor(net_, li, MYEA_TENSOR_NORM_VARIANCES_AVERAGES | sel, norm_variances_averages_[li].data() + dg * per, per))) return false;
                }
                continue;
            }
            if (!Ok("Set__HIP", myea_hip_upload_tensor(net_, li, MYEA_TENSOR_NORM_MEANS_AVERAGES, norm_means_averages_[li].data(), norm_means_averages_[li].size())) ||
                !Ok("Set__HIP", myea_hip_upload_tensor(net_, li, MYEA_TENSOR_NORM_VARIANCES_AVERAGES, norm_variances_averages_[li].data(), norm_variances_averages_[li].size()))) return false;
        }
        return Copy__Parameters__Host_To_Device() && Copy__Dropout_Mask__Host_To_Device();
    }
    // The reference's checkpoint: Save_General_Parameters / Save_Dimension_Parameters (Neural_Network__Save.cpp:23-624) write the
    // two text files, Load (Neural_Network__Load.cpp:2323) reads them back; see myea_nn_hip_io.hpp.  Saving with a device object
    // first pulls the parameters and the normalisation running statistics from the device; after Load the caller picks the batch
    // size (Update__Batch_Size) and calls Set__HIP(true).
    bool Save_General_Parameters(std::string const &path);
    bool Save_Dimension_Parameters(std::string const &path);
    bool Load(std::string const &path_dimension, std::string const &path_parameters, size_t maximum_allowable_memory = 0);
    bool Use__HIP() const { return net_ != nullptr; }

    // Data.hpp:3119-3189
    bool Copy__Parameters__Host_To_Device() { return Need("Copy__Parameters__Host_To_Device") && Ok("Copy__Parameters__Host_To_Device", myea_hip_upload_parameters(net_, ptr_array_parameters, total_parameters)); }
    bool Copy__Parameters__Device_To_Host() { return Need("Copy__Parameters__Device_To_Host") && Ok("Copy__Parameters__Device_To_Host", myea_hip_download_parameters(net_, ptr_array_parameters, total_parameters)); }
    bool Copy__Optimizer__Device_To_Host(int kind, T_ *dst) { return Need("Copy__Optimizer__Device_To_Host") && Ok("Copy__Optimizer__Device_To_Host", myea_hip_download_optimizer_state(net_, kind, dst, total_parameters)); }
    bool Copy__Optimizer__Host_To_Device(int kind, T_ const *src) { return Need("Copy__Optimizer__Host_To_Device") && Ok("Copy__Optimizer__Host_To_Device", myea_hip_upload_optimizer_state(net_, kind, src, total_parameters)); }
    bool Copy__Derivatives_Parameters__Device_To_Host(T_ *dst) { return Need("Copy__Derivatives_Parameters__Device_To_Host") && Ok("Copy__Derivatives_Parameters__Device_To_Host", myea_hip_download_gradient(net_, dst, total_parameters)); }
    // zoneout masks as the caller's Dropout_Zoneout() leaves them in ptr_array_cell_units_mask_dropout_zoneout:
    // [state | output] halves, per LSTM layer [T][cells] (Neural_Network.cpp:3964-3995); `count` = 2 x T x total cells
    bool Copy__Zoneout_Mask__Host_To_Device(bool const *ptr_array_cell_units_mask_dropout_zoneout, size_t count)
    {
        if (!Need("Copy__Zoneout_Mask__Host_To_Device")) return false;
        std::vector<uint8_t> bytes(count);
        for (size_t i = 0; i < count; ++i) bytes[i] = ptr_array_cell_units_mask_dropout_zoneout[i] ? 1 : 0;
        return Ok("Copy__Zoneout_Mask__Host_To_Device", myea_hip_upload_zoneout_masks(net_, bytes.data(), bytes.size()));
    }
    bool Copy__Dropout_Mask__Host_To_Device()
    {
        if (!Need("Copy__Dropout_Mask__Host_To_Device")) return false;
        std::vector<uint8_t> bytes(desc_.total_mask_units);
        for (size_t i = 0; i < bytes.size(); ++i) bytes[i] = ptr_array_units_mask_dropout_bernoulli[i] ? 1 : 0;
        return Ok("Copy__Dropout_Mask__Host_To_Device", myea_hip_upload_masks(net_, bytes.data(), bytes.size()));
    }

    // Train.cpp:93-263
    void Clear_Training_Arrays()
    {
        if (!Need("Clear_Training_Arrays") || !PushFields("Clear_Training_Arrays")) return;
        if (Ok("Clear_Training_Arrays", myea_hip_clear_training_arrays(net_))) PullState();
    }
    void Reset__Loss() { if (Need("Reset__Loss")) Ok("Reset__Loss", myea_hip_reset_loss(net_)); }

    // ---- the five step entry points (Data.hpp:2896, 1033, 1709, 2199, 849) ----
    // The reference's training loop calls them from inside `#pragma omp parallel` (Dataset.cpp:645-658): every thread of the
    // team makes the same call and the work is shared inside.  Here one thread - the master - makes the device call, between
    // two barriers, so the unchanged loop may keep its parallel region; outside a parallel region the barriers do nothing.
    // input_layer_index / output_layer_index: only the defaults (the whole network) are on this path.
    void Forward_Pass(size_t batch_size_received, T_ const *const *ptr_array_inputs, long long int input_layer_index_received = -1ll,
                      long long int output_layer_index_received = -1ll)
    {
        Solo([&] {
            if (input_layer_index_received != -1ll || output_layer_index_received != -1ll) { Fail("Forward_Pass", "a forward pass over a range of layers is not on this path"); return; }
            if (!Need("Forward_Pass") || !PushFields("Forward_Pass")) return;
            const size_t row = (size_t)desc_.layers[0].n_units * desc_.number_recurrent_depth;
            if (!Flatten("Forward_Pass", batch_size_received, ptr_array_inputs, row)) return;
            Ok("Forward_Pass", myea_hip_forward_pass(net_, batch_size_received, rows_.data(), 0));
        });
    }
    void Compute__Error(size_t batch_size_received, T_ const *const *ptr_array_desireds_outputs)
    {
        Solo([&] {
            if (!Need("Compute__Error") || !PushFields("Compute__Error")) return;
            const size_t row = (size_t)desc_.layers[desc_.n_layers - 1].n_units * desc_.number_recurrent_depth;
            if (!Flatten("Compute__Error", batch_size_received, ptr_array_desireds_outputs, row)) return;
            Ok("Compute__Error", myea_hip_compute_error(net_, batch_size_received, rows_.data(), 0));
        });
    }
    void Backward_Pass(size_t batch_size_received)
    {
        Solo([&] { if (Need("Backward_Pass") && PushFields("Backward_Pass")) Ok("Backward_Pass", myea_hip_backward_pass(net_, batch_size_received)); });
    }
    // Backward_Pass and Update_Derivative_Weight(batch, 1, total_layers) of Train_Batch_BP (Dataset.cpp:645-658) as one call
    void Backward_Pass__Update_Derivative_Weight(size_t batch_size_received)
    {
        Solo([&] { if (Need("Backward_Pass") && PushFields("Backward_Pass")) Ok("Backward_Pass", myea_hip_backward_pass_and_update_derivative_weight(net_, batch_size_received)); });
    }
    // Data.hpp:2199: the layers [ptr_layer_it_received, ptr_layer_end_received) of ptr_array_layers
    void Update_Derivative_Weight(size_t batch_size_received, struct Layer *const ptr_layer_it_received, struct Layer const *const ptr_layer_end_received)
    {
        if (ptr_array_layers == nullptr || ptr_layer_it_received < ptr_array_layers || ptr_layer_end_received > ptr_last_layer || ptr_layer_it_received > ptr_layer_end_received) {
            Solo([&] { Fail("Update_Derivative_Weight", "the layer pointers do not lie in ptr_array_layers"); });
            return;
        }
        Update_Derivative_Weight(batch_size_received, (size_t)(ptr_layer_it_received - ptr_array_layers), (size_t)(ptr_layer_end_received - ptr_array_layers));
    }
    // the same with layer indices; end_layer_index 0 = the last layer
    void Update_Derivative_Weight(size_t batch_size_received, size_t first_layer_index = 1, size_t end_layer_index = 0)
    {
        Solo([&] {
            if (!Need("Update_Derivative_Weight")) return;
            Ok("Update_Derivative_Weight", myea_hip_update_derivative_weight(net_, batch_size_received, first_layer_index, end_layer_index ? end_layer_index : desc_.n_layers));
        });
    }
    void Update_Parameter(size_t batch_size_received, size_t training_size_received)
    {
        Solo([&] {
            if (!Need("Update_Parameter") || !PushFields("Update_Parameter")) return;
            Ok("Update_Parameter", myea_hip_update_parameter(net_, batch_size_received, training_size_received));
            PullState();
        });
    }
    // Backward_Pass, Update_Derivative_Weight(batch, 1, total_layers) and Update_Parameter as one call (Dataset.cpp:645-658 and
    // :7652-7658): the update of a layer's weights may then run beside the contractions of the layers below it
    void Backward_Pass__Update_Derivative_Weight__Update_Parameter(size_t batch_size_received, size_t training_size_received)
    {
        Solo([&] {
            if (!Need("Backward_Pass") || !PushFields("Backward_Pass")) return;
            Ok("Backward_Pass", myea_hip_backward_pass_update_derivative_weight_and_update_parameter(net_, batch_size_received, training_size_received));
            PullState();
        });
    }

    // Dropout_Bernoulli (Data.hpp:944; Neural_Network__Dropout__Bernoulli__Loop.cpp:33-97): new keep / drop draws for the
    // layers whose dropout is BERNOULLI - never BERNOULLI_INVERTED, which has its own function there - in layer order (the
    // input layer first, the output layer never), per layer [time step][unit], one std::bernoulli_distribution(retention
    // probability) draw from a std::mt19937 each (Common_Library Random/Bernoulli.hpp); a retention probability of 0 clears
    // the layer's masks.  The masks then go to the device when there is one.
    void Dropout_Bernoulli(void)
    {
        Solo([&] {
            bool any = false;
            for (size_t li = 0; li + 1 < desc_.n_layers; ++li) {
                const myea_layer_desc &l = desc_.layers[li];
                if (l.type_dropout != MYEA_DROPOUT_BERNOULLI) continue;
                const size_t first = l.first_mask_index;
                const size_t end = li + 1 < desc_.n_layers ? desc_.layers[li + 1].first_mask_index : desc_.total_mask_units;
                if (end == first) { if (li != 0) Fail("Dropout_Bernoulli", "the layer type is not managed (no activation unit)"); continue; }
                any = true;
                const T_ keep = l.dropout_values[0];
                if (keep != 0.f) {
                    if (bernoulli_probability_ != keep) { bernoulli_probability_ = keep; bernoulli_.param(std::bernoulli_distribution::param_type(keep)); }
                    for (size_t i = first; i < end; ++i) ptr_array_units_mask_dropout_bernoulli[i] = bernoulli_(bernoulli_generator_);
                } else {
                    for (size_t i = first; i < end; ++i) ptr_array_units_mask_dropout_bernoulli[i] = false;
                }
            }
            if (any && net_) Copy__Dropout_Mask__Host_To_Device();
        });
    }
    // Base::Seed of the reference's generator classes
    void Set__Seed__Dropout_Bernoulli(unsigned int seed) { bernoulli_generator_.seed(seed); bernoulli_.reset(); }

    // Compute__Loss (Neural_Network__Compute__Loss__Loop.cpp:22): loss / accuracy of the last forward pass, no delta
    void Compute__Loss(size_t batch_size_received, T_ const *const *ptr_array_desireds_outputs)
    {
        if (!Need("Compute__Loss") || !PushFields("Compute__Loss")) return;
        const size_t row = (size_t)desc_.layers[desc_.n_layers - 1].n_units * desc_.number_recurrent_depth;
        if (!Flatten("Compute__Loss", batch_size_received, ptr_array_desireds_outputs, row)) return;
        Ok("Compute__Loss", myea_hip_compute_loss(net_, batch_size_received, rows_.data(), 0));
    }
    // Compute__Accuracy__R (Neural_Network__Compute__R__Loop.cpp:22): the means are ptr_array_accuracy_values[0] / [1],
    // which Dataset::Measure_Accuracy has divided by the number of entries (R_Means)
    void Compute__Accuracy__R(size_t batch_size_received, T_ const *const *ptr_array_desireds_outputs)
    {
        if (!Need("Compute__Accuracy__R") || !PushFields("Compute__Accuracy__R")) return;
        const size_t row = (size_t)desc_.layers[desc_.n_layers - 1].n_units * desc_.number_recurrent_depth;
        if (!Flatten("Compute__Accuracy__R", batch_size_received, ptr_array_desireds_outputs, row)) return;
        Ok("Compute__Accuracy__R", myea_hip_compute_accuracy_r(net_, batch_size_received, rows_.data(), 0, r_mean_desired_, r_mean_predicted_));
    }
    // device-resident variants: [batch][T * width] rows already in HBM (a dataset kept on the GPU)
    void Forward_Pass__Device(size_t B, T_ const *dev) { if (Need("Forward_Pass") && PushFields("Forward_Pass")) Ok("Forward_Pass", myea_hip_forward_pass(net_, B, dev, 1)); }
    void Compute__Error__Device(size_t B, T_ const *dev) { if (Need("Compute__Error") && PushFields("Compute__Error")) Ok("Compute__Error", myea_hip_compute_error(net_, B, dev, 1)); }
    void Compute__Loss__Device(size_t B, T_ const *dev) { if (Need("Compute__Loss") && PushFields("Compute__Loss")) Ok("Compute__Loss", myea_hip_compute_loss(net_, B, dev, 1)); }
    void Compute__Accuracy__R__Device(size_t B, T_ const *dev)
    { if (Need("Compute__Accuracy__R") && PushFields("Compute__Accuracy__R")) Ok("Compute__Accuracy__R", myea_hip_compute_accuracy_r(net_, B, dev, 1, r_mean_desired_, r_mean_predicted_)); }
    // the in-place division of the two running sums in Dataset::Measure_Accuracy (Dataset.cpp:7712-7713)
    void R_Means(size_t number_entries)
    {
        myea_loss_state s;
        if (!Get__Loss_State(&s) || number_entries == 0) return;
        r_mean_desired_ = (T_)(s.accuracy_value / (double)number_entries);
        r_mean_predicted_ = (T_)(s.accuracy_r[0] / (double)number_entries);
    }

    // Get__Loss (Neural_Network__Loss.cpp:103-214) / Get__Accuracy (Neural_Network__Accuracy.cpp:88-113); dataset kinds as
    // Enum_Type_Dataset.hpp: 0 none (read the counters), 1 testing, 2 training, 3 validation (the stored values)
    enum { TYPE_DATASET_NONE = 0, TYPE_DATASET_TESTING = 1, TYPE_DATASET_TRAINING = 2, TYPE_DATASET_VALIDATION = 3 };
    T_ loss_training = FLT_MAX, loss_validating = FLT_MAX, loss_testing = FLT_MAX;
    T_ accuracy_training = 0.f, accuracy_validating = 0.f, accuracy_testing = 0.f;
    size_t number_accuracy_trial = 0;
    size_t Get__Output_Size() const { return desc_.layers[desc_.n_layers - 1].n_units; }
    T_ Get__Loss(unsigned int type_dataset = TYPE_DATASET_NONE)
    {
        switch (type_dataset) {
        case TYPE_DATASET_TRAINING: return loss_training;
        case TYPE_DATASET_VALIDATION: return loss_validating;
        case TYPE_DATASET_TESTING: return loss_testing;
        case TYPE_DATASET_NONE: break;
        default: return 1.f;
        }
        myea_loss_state s;
        if (!Get__Loss_State(&s)) return 1.f;
        const double n = (double)s.number_loss;
        switch (type_loss_function) {
        case MYEA_LOSS_L1: case MYEA_LOSS_L2: return (T_)s.loss_values;
        case MYEA_LOSS_ME: case MYEA_LOSS_MAE: case MYEA_LOSS_MSE: case MYEA_LOSS_MAPE: case MYEA_LOSS_SMAPE:
            return s.number_loss ? (T_)(s.loss_values / n) : 1.f;
        case MYEA_LOSS_RMSE: return s.number_loss ? (T_)std::sqrt(s.loss_values / n) : 1.f;
        case MYEA_LOSS_CROSS_ENTROPY: return s.number_loss ? (T_)(s.loss_values / (double)(s.number_loss / Get__Output_Size())) : FLT_MAX;
        case MYEA_LOSS_BIT: return (T_)s.number_bit_fail;
        default: return 1.f;
        }
    }
    T_ Get__Accuracy(unsigned int type_dataset = TYPE_DATASET_NONE)
    {
        switch (type_dataset) {
        case TYPE_DATASET_TRAINING: return accuracy_training;
        case TYPE_DATASET_VALIDATION: return accuracy_validating;
        case TYPE_DATASET_TESTING: return accuracy_testing;
        case TYPE_DATASET_NONE: break;
        default: return 0.f;
        }
        myea_loss_state s;
        if (!Get__Loss_State(&s)) return 0.f;
        if (type_accuracy_function == MYEA_ACCURACY_R) {
            const double den = s.accuracy_r[2] * s.accuracy_r[3];
            const double r = den == 0.0 ? 0.0 : s.accuracy_r[1] / (std::sqrt(s.accuracy_r[2]) * std::sqrt(s.accuracy_r[3]));
            return (T_)(r < -1.0 ? -1.0 : (r > 1.0 ? 1.0 : r));
        }
        return number_accuracy_trial == 0 ? 0.f : (T_)(s.accuracy_value / (double)number_accuracy_trial * 100.0);
    }
    void Set__Loss(unsigned int type_dataset, T_ v)
    {
        if (type_dataset == TYPE_DATASET_TRAINING) loss_training = v; else if (type_dataset == TYPE_DATASET_VALIDATION) loss_validating = v;
        else if (type_dataset == TYPE_DATASET_TESTING) loss_testing = v; else std::printf("Set__Loss: ERROR: Loss type (%u) is not managed in the switch.\n", type_dataset);
    }
    void Set__Accuracy(unsigned int type_dataset, T_ v)
    {
        if (type_dataset == TYPE_DATASET_TRAINING) accuracy_training = v; else if (type_dataset == TYPE_DATASET_VALIDATION) accuracy_validating = v;
        else if (type_dataset == TYPE_DATASET_TESTING) accuracy_testing = v; else std::printf("Set__Accuracy: ERROR: Accuracy type (%u) is not managed in the switch.\n", type_dataset);
    }
    bool Get__Loss_State(myea_loss_state *out) { return Need("Get__Loss_State") && Ok("Get__Loss_State", myea_hip_get_loss(net_, out)); }

    myea_net_desc const &Get__Descriptor() const { return desc_; }
    myea_hip_net *Get__Device_Handle() { return net_; }

private:
    myea_net_desc desc_;
    myea_hip_net *net_ = nullptr;
    std::vector<Layer> layers_;
    std::mt19937 bernoulli_generator_{5489u};
    std::bernoulli_distribution bernoulli_{0.5};
    T_ bernoulli_probability_ = 0.5f;
    myea_hyper pushed_;              // what the device object last received from the public fields
    bool pushed_valid_ = false;
    unsigned int pushed_state_ = 0;

    // one thread of the calling team runs f, the others wait for it (see the step entry points)
    template <class F>
    static void Solo(F &&f)
    {
#ifdef _OPENMP
#pragma omp barrier
#pragma omp master
        f();
#pragma omp barrier
#else
        f();
#endif
    }
    void RefreshLayers()
    {
        layers_.assign(desc_.n_layers, Layer());
        for (size_t i = 0; i < desc_.n_layers; ++i) {
            const myea_layer_desc &l = desc_.layers[i];
            layers_[i].type_layer = l.type_layer; layers_[i].type_dropout = l.type_dropout; layers_[i].use_bidirectional = l.use_bidirectional != 0;
            for (int k = 0; k < 2; ++k) layers_[i].dropout_values[k] = l.dropout_values[k];
        }
        total_layers = desc_.n_layers;
        ptr_array_layers = layers_.empty() ? nullptr : layers_.data();
        ptr_last_layer = ptr_array_layers ? ptr_array_layers + total_layers : nullptr;
    }
    std::vector<T_> rows_;
    std::vector<std::vector<T_>> norm_means_averages_, norm_variances_averages_;   // per layer [T][units] ([direction][group][T][K] for an LSTM layer), from a checkpoint
    T_ r_mean_desired_ = 0.f, r_mean_predicted_ = 0.f;

    static bool Fail(const char *fn, const char *what) { std::printf("%s: ERROR: %s.\n", fn, what); return false; }
    bool Ok(const char *fn, int rc) { if (rc != MYEA_OK) { Fail(fn, myea_hip_last_error()); return false; } return true; }
    bool Need(const char *fn) const { if (!net_) { Fail(fn, "the device object is not initialised (Set__HIP)"); return false; } return true; }
    bool CheckLayer(const char *fn, size_t i) const
    {
        if (i == 0 || i >= desc_.n_layers) return Fail(fn, "layer index overflow");
        return true;
    }
    // a structural change after Set__HIP needs a new device object, as a changed Layer does in the reference's CUDA path
    bool Dirty() { if (net_) { myea_hip_destroy(net_); net_ = nullptr; } pushed_valid_ = false; RefreshLayers(); return true; }
    void Deallocate()
    {
        if (net_) { myea_hip_destroy(net_); net_ = nullptr; }
        delete[] ptr_array_parameters; ptr_array_parameters = nullptr;
        delete[] ptr_array_units_mask_dropout_bernoulli; ptr_array_units_mask_dropout_bernoulli = nullptr;
        norm_means_averages_.clear(); norm_variances_averages_.clear();
        layers_.clear(); ptr_array_layers = nullptr; ptr_last_layer = nullptr; total_layers = 0; pushed_valid_ = false;
    }
    bool Relayout(const char *fn)
    {
        Dirty();
        const size_t old_p = total_parameters;
        T_ *old = ptr_array_parameters;
        if (myea_net_desc_layout(&desc_) != MYEA_OK) return Fail(fn, "the layer list is not valid on this path");
        total_parameters = desc_.total_parameters; total_weights = desc_.total_weights; total_bias = desc_.total_bias;
        ptr_array_parameters = new T_[total_parameters ? total_parameters : 1]();
        if (old) std::memcpy(ptr_array_parameters, old, sizeof(T_) * (old_p < total_parameters ? old_p : total_parameters));
        // scales start at one (Allocate__Parameter__Normalization), shifts at zero
        if (desc_.total_normalized_units && old_p <= desc_.total_weights + desc_.total_bias)
            for (size_t i = 0; i < desc_.total_normalized_units; ++i) ptr_array_parameters[desc_.total_weights + desc_.total_bias + i] = 1.f;
        delete[] old;
        delete[] ptr_array_units_mask_dropout_bernoulli;
        ptr_array_units_mask_dropout_bernoulli = new bool[desc_.total_mask_units ? desc_.total_mask_units : 1];
        for (size_t i = 0; i < desc_.total_mask_units; ++i) ptr_array_units_mask_dropout_bernoulli[i] = true;
        RefreshLayers();
        return true;
    }
    void PullState()
    {
        myea_hyper h;
        if (myea_hip_get_hyper(net_, &h) != MYEA_OK) return;
        optimizer_time_step = h.optimizer_time_step; epoch_time_step = h.epoch_time_step; adam_previous_beta2 = h.adam_previous_beta2;
        loss_rprop = h.loss_rprop; previous_loss_rprop = h.previous_loss_rprop;
        warm_restarts_maximum_learning_rate = h.warm_restarts_maximum_learning_rate; warm_restarts_T_i = h.warm_restarts_T_i;
        // the device object and the public fields agree again: nothing to push until the caller writes a field
        if (pushed_valid_) { std::memset(&pushed_, 0, sizeof(pushed_)); AssignFields(pushed_); }
    }
    // the public fields written into a myea_hyper
    void AssignFields(myea_hyper &h) const
    {
        h.type_optimizer_function = type_optimizer_function; h.type_loss_function = type_loss_function; h.type_accuracy_function = type_accuracy_function;
        h.use_Nesterov = use_Nesterov; h.use_adam_bias_correction = use_adam_bias_correction; h.use_clip_gradient = use_clip_gradient;
        h.learning_rate = learning_rate; h.learning_rate_final = learning_rate_final; h.learning_momentum = learning_momentum; h.learning_gamma = learning_gamma;
        h.adam_learning_rate = adam_learning_rate; h.adam_beta1 = adam_beta1; h.adam_beta2 = adam_beta2; h.adam_epsilon = adam_epsilon;
        h.regularization__weight_decay = regularization__weight_decay; h.clip_gradient = clip_gradient; h.accuracy_variance = accuracy_variance;
        h.bit_fail_limit = bit_fail_limit; h.normalization_momentum_average = normalization_momentum_average; h.normalization_epsilon = normalization_epsilon;
        h.batch_renormalization_r_correction_maximum = batch_renormalization_r_correction_maximum;
        h.batch_renormalization_d_correction_maximum = batch_renormalization_d_correction_maximum;
        h.number_time_delays = (uint32_t)number_time_delays;
        h.use_normalized_weight_decay = use_normalized_weight_decay; h.use_Warm_Restarts = use_Warm_Restarts;
        h.adam_gamma = adam_gamma; h.regularization__max_norm_constraints = regularization__max_norm_constraints;
        h.rprop_increase_factor = rprop_increase_factor; h.rprop_decrease_factor = rprop_decrease_factor;
        h.rprop_delta_min = rprop_delta_min; h.rprop_delta_max = rprop_delta_max; h.rprop_delta_zero = rprop_delta_zero;
        h.warm_restarts_decay_learning_rate = warm_restarts_decay_learning_rate;
        h.warm_restarts_minimum_learning_rate = warm_restarts_minimum_learning_rate; h.warm_restarts_multiplier = warm_restarts_multiplier;
        h.optimizer_time_step = optimizer_time_step; h.epoch_time_step = epoch_time_step; h.adam_previous_beta2 = adam_previous_beta2;
        h.loss_rprop = loss_rprop; h.previous_loss_rprop = previous_loss_rprop;
        h.warm_restarts_maximum_learning_rate = warm_restarts_maximum_learning_rate; h.warm_restarts_T_i = warm_restarts_T_i;
    }
    // The public fields go to the device object when one of them differs from what it last received (a step function is
    // called four times per batch; the fields change between epochs at most).  Fields of the library's state that this class
    // does not hold are read back first, so a push never overwrites them.
    bool PushFields(const char *fn)
    {
        myea_hyper want;
        std::memset(&want, 0, sizeof(want));
        AssignFields(want);
        if (!pushed_valid_ || std::memcmp(&want, &pushed_, sizeof(want)) != 0) {
            myea_hyper h;
            if (myea_hip_get_hyper(net_, &h) != MYEA_OK) return Fail(fn, myea_hip_last_error());
            AssignFields(h);
            if (myea_hip_set_hyper(net_, &h) != MYEA_OK) return Fail(fn, myea_hip_last_error());
            pushed_ = want;
        }
        if (!pushed_valid_ || pushed_state_ != type_state_propagation) {
            if (!Ok(fn, myea_hip_set_state_propagation(net_, type_state_propagation))) return false;
            pushed_state_ = type_state_propagation;
        }
        pushed_valid_ = true;
        return true;
    }
    bool Flatten(const char *fn, size_t B, T_ const *const *rows, size_t row)
    {
        if (rows == nullptr) return Fail(fn, "null row pointer array");
        if (B > desc_.batch_size) { std::printf("%s: ERROR: Overflow of memory. Unable to process %zu examples out of %u allocated.\n", fn, B, desc_.batch_size); return false; }
        rows_.resize(B * row);
        for (size_t b = 0; b < B; ++b) std::memcpy(rows_.data() + b * row, rows[b], row * sizeof(T_));
        return true;
    }
};

}  // namespace MyEA_HIP

#include "myea_nn_hip_io.hpp"

