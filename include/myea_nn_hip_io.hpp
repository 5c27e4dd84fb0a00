// myea_nn_hip_io.hpp — the reference's two checkpoint text files, written and read by Neural_Network_HIP.
//
// `Save_General_Parameters` (Neural_Network__Save.cpp:23-202) holds the hyper-parameters, `Save_Dimension_Parameters`
// (:204-624) the structure, every weight with its flat index, the normalisation scales / shifts / running statistics
// and the per-unit activation functions.  The token order below is the writer's, which the reference's loader
// (Neural_Network__Load.cpp:82-2321, 2323-6882) consumes strictly in sequence; a file written here is meant to load there
// and the other way round.  The reference ships no checkpoint file to compare with: the format is followed by reading.
//
// Fields the reference writes and this path does not hold (QuickProp, SARProp, L1 / L2 / SRIP, tied parameters, coded
// dropout, the CPU thread settings) are written at the reference's defaults and skipped when read.
// Included by myea_nn_hip.hpp; not a header of its own.
#pragma once

#include <cstdlib>
#include <fstream>
#include <iomanip>
#include <sstream>
#include <string>

namespace MyEA_HIP {

namespace io_detail {

// MyEA::String::To_string<T_, DEFAULTFLOAT> (Common_Library/include/Strings/String.hpp:103-121): 16 significant digits
inline std::string TS(double v, unsigned precision = 16u)
{
    std::ostringstream o;
    o << std::defaultfloat << std::setprecision((int)precision) << v;
    return o.str();
}
inline std::string TS(float v) { std::ostringstream o; o << std::defaultfloat << std::setprecision(16) << v; return o.str(); }

// Activation_Function__To__Class_Activation_Function (Train.cpp:453-500): ENUM_TYPE_LAYER_ACTIVATION of a function
inline unsigned Class_Activation(unsigned af)
{
    switch (af) {
    case MYEA_AF_COSINE_SYMMETRIC: case MYEA_AF_ELLIOT_SYMMETRIC: case MYEA_AF_GAUSSIAN_SYMMETRIC: case MYEA_AF_LINEAR_PIECE_SYMMETRIC:
    case MYEA_AF_SINE_SYMMETRIC: case MYEA_AF_TANH: case MYEA_AF_TANH_STEPWISE: case MYEA_AF_THRESHOLD_SYMMETRIC: return 5u;   // SYMMETRIC
    case MYEA_AF_LEAKY_RELU: case MYEA_AF_PARAMETRIC_RELU: case MYEA_AF_RELU: return 2u;                                        // RECTIFIER
    case MYEA_AF_SELU: return 3u;                                                                                                // SELF_NORMALIZATION
    case MYEA_AF_SOFTMAX: return 4u;
    case MYEA_AF_NONE: return 0u;
    default: return 1u;                                                                                                          // ASYMMETRIC
    }
}

// whitespace-separated tokens of a file, consumed front to back
struct Tokens {
    std::vector<std::string> t;
    size_t at = 0;
    bool Read(std::string const &path)
    {
        std::ifstream f(path, std::ios::in | std::ios::binary);
        if (!f.is_open()) return false;
        std::string w;
        while (f >> w) t.push_back(w);
        return true;
    }
    // the value after the next token equal to `key`; false when the key does not come
    bool Value(const char *key, std::string *out)
    {
        for (size_t i = at; i + 1 < t.size(); ++i)
            if (t[i] == key) { *out = t[i + 1]; at = i + 2; return true; }
        return false;
    }
    bool Size(const char *key, size_t *out) { std::string v; if (!Value(key, &v)) return false; *out = (size_t)std::strtoull(v.c_str(), nullptr, 10); return true; }
    bool Real(const char *key, float *out) { std::string v; if (!Value(key, &v)) return false; *out = std::strtof(v.c_str(), nullptr); return true; }
    bool Bool(const char *key, bool *out) { size_t v; if (!Size(key, &v)) return false; *out = v != 0; return true; }
    // the next "weight[<index>] <value>" pair
    bool Weight(size_t *index, float *value)
    {
        for (size_t i = at; i + 1 < t.size(); ++i)
            if (t[i].compare(0, 7, "weight[") == 0) {
                *index = (size_t)std::strtoull(t[i].c_str() + 7, nullptr, 10);
                *value = std::strtof(t[i + 1].c_str(), nullptr);
                at = i + 2;
                return true;
            }
        return false;
    }
    // the next token is expected to start with `prefix` ("Neuron_unit[", "Hidden", ...)
    bool Skip(const char *prefix)
    {
        const size_t n = std::strlen(prefix);
        for (size_t i = at; i < t.size(); ++i)
            if (t[i].compare(0, n, prefix) == 0) { at = i + 1; return true; }
        return false;
    }
};

}  // namespace io_detail

inline bool Neural_Network_HIP::Save_General_Parameters(std::string const &path)
{
    using io_detail::TS;
    std::string s;
    auto line = [&s](std::string const &k, std::string const &v) { s += k + " " + v + "\n"; };
    auto str = [](size_t v) { return std::to_string(v); };
    s += "|===| GRADIENT DESCENT PARAMETERS |===|\n";
    line("learning_rate", TS(learning_rate)); line("learning_rate_final", TS(learning_rate_final)); line("learning_momentum", TS(learning_momentum));
    line("learning_gamma", TS(learning_gamma)); line("use_Nesterov", str(use_Nesterov));
    s += "|END| GRADIENT DESCENT PARAMETERS |END|\n\n|===| QUICKPROP PARAMETERS |===|\n";
    line("quickprop_decay", TS(-0.0001f)); line("quickprop_mu", TS(1.75f));
    s += "|END| QUICKPROP PARAMETERS |END|\n\n|===| RESILLENT PROPAGATION PARAMETERS |===|\n";
    line("rprop_increase_factor", TS(rprop_increase_factor)); line("rprop_decrease_factor", TS(rprop_decrease_factor)); line("rprop_delta_min", TS(rprop_delta_min));
    line("rprop_delta_max", TS(rprop_delta_max)); line("rprop_delta_zero", TS(rprop_delta_zero));
    s += "|END| RESILLENT PROPAGATION PARAMETERS |END|\n\n|===| SARPROP PARAMETERS |===|\n";
    line("sarprop_weight_decay_shift", TS(-6.644f)); line("sarprop_step_error_threshold_factor", TS(0.1f)); line("sarprop_step_error_shift", TS(1.385f));
    line("sarprop_temperature", TS(0.015f)); line("sarprop_epoch", "0");
    s += "|END| SARPROP PARAMETERS |END|\n\n|===| ADAM PARAMETERS |===|\n";
    line("adam_learning_rate", TS(adam_learning_rate)); line("adam_beta1", TS(adam_beta1)); line("adam_beta2", TS(adam_beta2)); line("adam_epsilon", TS(adam_epsilon));
    line("adam_bias_correction", str(use_adam_bias_correction)); line("adam_gamma", TS(adam_gamma));
    s += "|END| ADAM PARAMETERS |END|\n\n|===| WARM RESTARTS PARAMETERS |===|\n";
    line("use_Warm_Restarts", str(use_Warm_Restarts)); line("warm_restarts_decay_learning_rate", TS(warm_restarts_decay_learning_rate));
    line("warm_restarts_maximum_learning_rate", TS(warm_restarts_initial_maximum_learning_rate)); line("warm_restarts_minimum_learning_rate", TS(warm_restarts_minimum_learning_rate));
    line("warm_restarts_initial_T_i", str((size_t)warm_restarts_initial_T_i)); line("warm_restarts_multiplier", str((size_t)warm_restarts_multiplier));
    s += "|END| WARM RESTARTS PARAMETERS |END|\n\n|===| TRAINING PARAMETERS |===|\n";
    line("type_optimizer_function", str(type_optimizer_function)); line("type_loss_function", str(type_loss_function)); line("type_accuracy_function", str(type_accuracy_function));
    line("bit_fail_limit", TS(bit_fail_limit)); line("pre_training_level", "0"); line("use_clip_gradient", str(use_clip_gradient)); line("clip_gradient", TS(clip_gradient));
    s += "|END| TRAINING PARAMETERS |END|\n\n|===| REGULARIZATION PARAMETERS |===|\n";
    line("regularization__max_norm_constraints", TS(regularization__max_norm_constraints)); line("regularization__l1", "0"); line("regularization__l2", "0");
    line("regularization__srip", "0"); line("regularization__weight_decay", TS(regularization__weight_decay)); line("use_normalized_weight_decay", str(use_normalized_weight_decay));
    s += "|END| REGULARIZATION PARAMETERS |END|\n\n|===| NORMALIZATION PARAMETERS |===|\n";
    line("normalization_momentum_average", TS(normalization_momentum_average)); line("normalization_epsilon", TS(normalization_epsilon));
    line("batch_renormalization_r_correction_maximum", TS(batch_renormalization_r_correction_maximum));
    line("batch_renormalization_d_correction_maximum", TS(batch_renormalization_d_correction_maximum));
    s += "|END| NORMALIZATION PARAMETERS |END|\n\n|===| LOSS PARAMETERS |===|\n";
    line("loss_training", TS(loss_training)); line("loss_validating", TS(loss_validating)); line("loss_testing", TS(loss_testing));
    s += "|END| LOSS PARAMETERS |END|\n\n|===| ACCURANCY PARAMETERS |===|\n";
    line("accuracy_variance", TS(accuracy_variance)); line("accuracy_training", TS(accuracy_training)); line("accuracy_validating", TS(accuracy_validating));
    line("accuracy_testing", TS(accuracy_testing));
    s += "|END| ACCURANCY PARAMETERS |END|\n\n|===| COMPUTATION PARAMETERS |===|\n";
    line("use_CUDA", "0"); line("use_OpenMP", "0"); line("percentage_maximum_thread_usage", TS(100.0, 9u)); line("maximum_batch_size", str(batch_size));
    s += "|END| COMPUTATION PARAMETERS |END|\n";
    std::ofstream f(path, std::ios::out | std::ios::binary);
    if (!f.is_open()) return Fail("Save_General_Parameters", "the file can not be opened");
    f.write(s.c_str(), (std::streamsize)s.size());
    f.flush();
    return f.fail() ? Fail("Save_General_Parameters", "write failed") : true;
}

inline bool Neural_Network_HIP::Save_Dimension_Parameters(std::string const &path)
{
    using io_detail::TS;
    const size_t L = desc_.n_layers, T = desc_.number_recurrent_depth;
    if (L < 2) return Fail("Save_Dimension_Parameters", "the network is not compiled");
    if (net_ && !Copy__Parameters__Device_To_Host()) return false;   // as the reference does under CUDA (:228-252)
    auto str = [](size_t v) { return std::to_string(v); };
    auto width = [this](size_t li) { return (size_t)myea_net_desc_number_outputs(&desc_, (uint32_t)li); };
    auto dirs = [this](size_t li) { return desc_.layers[li].use_bidirectional ? 2u : 1u; };
    // the reference's unit arrays: one global array per unit type, layers in order (Assign__Layer, Neural_Network__Compile.cpp:40-108)
    std::vector<size_t> neuron_at(L, 0), cell_at(L, 0), basic_at(L, 0), indice_at(L, 0), ind_at(L, 0), group(L, 0), af_units(L, 0), norm_units(L, 0);
    size_t n_basic = 0, n_indice = 0, n_neuron = 0, n_af = 0, n_ind = 0, n_block = 0, n_cell = 0, n_norm = 0;
    for (size_t li = 0; li < L; ++li) {
        const myea_layer_desc &l = desc_.layers[li];
        // a residual block's dense members (fully-connected or independently recurrent) keep their activation, recurrent and
        // normalised units on their input side: none on the block's first member, fan-in many on the others
        // (Assign__Post__Residual_Layer, Neural_Network__Compile.cpp:283-376)
        if (l.type_layer == MYEA_LAYER_RESIDUAL)
            for (size_t m = li + 1; m <= li + l.block_depth && m < L; ++m)
                if (desc_.layers[m].type_layer == MYEA_LAYER_FULLY_CONNECTED || desc_.layers[m].type_layer == MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT)
                    group[m] = m == li + 1 ? 1 : 2;
        const size_t H = width(li), In = li ? width(myea_net_desc_previous_layer(&desc_, (uint32_t)li)) : 0;
        neuron_at[li] = n_neuron; cell_at[li] = n_cell; basic_at[li] = n_basic; indice_at[li] = n_indice; ind_at[li] = n_ind;
        switch (l.type_layer) {
        case MYEA_LAYER_FULLY_CONNECTED:
            n_neuron += H; af_units[li] = group[li] == 0 ? H : (group[li] == 1 ? 0 : In); n_af += af_units[li]; norm_units[li] = group[li] == 0 ? H : In; break;
        case MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT:
            n_neuron += H; af_units[li] = group[li] == 0 ? H : (group[li] == 1 ? 0 : In); n_ind += af_units[li]; norm_units[li] = group[li] == 0 ? H : In; break;
        case MYEA_LAYER_LSTM: n_block += (size_t)l.n_units * dirs(li); n_cell += H * dirs(li); norm_units[li] = (3 * H + 6 * l.n_units) * dirs(li); break;
        case MYEA_LAYER_RESIDUAL: n_basic += H; norm_units[li] = width(li + l.block_depth); break;
        case MYEA_LAYER_AVERAGE_POOLING: n_basic += H; break;
        case MYEA_LAYER_MAX_POOLING: n_indice += H; break;
        default: return Fail("Save_Dimension_Parameters", "layer type is not managed");
        }
        n_norm += norm_units[li];
    }
    // running statistics of the normalised layers ([T][units]); ones and zeros while no device object exists
    std::vector<std::vector<float>> mean(L), var(L);
    size_t norm_at = 0;
    std::vector<size_t> first_norm(L, 0);
    for (size_t li = 0; li < L; ++li) {
        first_norm[li] = norm_at; norm_at += norm_units[li];
        if (desc_.layers[li].type_normalization == MYEA_NORMALIZATION_NONE || norm_units[li] == 0) continue;   // (a pooling layer owns no normalised unit, whatever its type says)
        mean[li].assign(T * norm_units[li], 0.f); var[li].assign(T * norm_units[li], 1.f);
        if (li < norm_means_averages_.size() && norm_means_averages_[li].size() == mean[li].size()) { mean[li] = norm_means_averages_[li]; var[li] = norm_variances_averages_[li]; }
        if (desc_.layers[li].type_layer == MYEA_LAYER_LSTM) {
            // a normalised LSTM layer (one cell per block): nine groups of K units per direction, held as [direction][group][T][K]
            if (desc_.layers[li].n_cells_per_block != 1) return Fail("Save_Dimension_Parameters", "a normalised LSTM layer needs one cell per block");
            const size_t K = desc_.layers[li].n_units;
            for (size_t dg = 0; net_ && dg < 9 * dirs(li); ++dg) {
                const int sel = MYEA_TENSOR_LSTM_NORM_GROUP((int)(dg % 9)) | (dg >= 9 ? MYEA_TENSOR_DIRECTION_BACKWARD : 0);
                if (myea_hip_download_tensor(net_, li, MYEA_TENSOR_NORM_MEANS_AVERAGES | sel, mean[li].data() + dg * T * K, T * K) != MYEA_OK ||
                    myea_hip_download_tensor(net_, li, MYEA_TENSOR_NORM_VARIANCES_AVERAGES | sel, var[li].data() + dg * T * K, T * K) != MYEA_OK)
                    return Fail("Save_Dimension_Parameters", myea_hip_last_error());
            }
            continue;
        }
        if (net_ && (myea_hip_download_tensor(net_, li, MYEA_TENSOR_NORM_MEANS_AVERAGES, mean[li].data(), mean[li].size()) != MYEA_OK ||
                     myea_hip_download_tensor(net_, li, MYEA_TENSOR_NORM_VARIANCES_AVERAGES, var[li].data(), var[li].size()) != MYEA_OK))
            return Fail("Save_Dimension_Parameters", myea_hip_last_error());
    }
    const float *P = ptr_array_parameters;
    const size_t scale_at = desc_.total_weights + desc_.total_bias, total_norm = desc_.total_normalized_units;

    std::string s;
    s.reserve(64 + 48 * (size_t)desc_.total_parameters);
    auto line = [&s](const char *indent, std::string const &k, std::string const &v) { s += indent; s += k; s += ' '; s += v; s += '\n'; };
    auto weight = [&](const char *indent, size_t index) { s += indent; s += "weight["; s += str(index); s += "] "; s += TS(P[index]); s += '\n'; };
    s += "|===| DIMENSION |===|\n";
    line("", "type_network", str(desc_.type_network)); line("", "number_layers", str(L)); line("", "number_recurrent_depth", str(T));
    line("", "number_time_delays", str(number_time_delays)); line("", "use_first_layer_as_input", "1"); line("", "use_last_layer_as_output", "1");
    line("", "total_basic_units", str(n_basic)); line("", "total_basic_indice_units", str(n_indice)); line("", "total_neuron_units", str(n_neuron));
    line("", "total_AF_units", str(n_af)); line("", "total_AF_Ind_recurrent_units", str(n_ind)); line("", "total_block_units", str(n_block));
    line("", "total_cell_units", str(n_cell)); line("", "total_normalized_units", str(n_norm)); line("", "total_parameters", str(desc_.total_parameters));
    line("", "total_weights", str(desc_.total_weights)); line("", "total_bias", str(desc_.total_bias));

    auto dropout = [&](const myea_layer_desc &l, bool hidden) {   // tmp_Get__Dropout__Parameters, :255-285
        line("    ", "type_dropout", str(l.type_dropout));
        if (hidden) line("      ", "use_coded_dropout", "0");
        float v0 = l.dropout_values[0];
        if (l.type_dropout == MYEA_DROPOUT_GAUSSIAN) v0 = v0 / (v0 + 1.f);   // back to the probability
        line("      ", "dropout_values[0]", TS(v0)); line("      ", "dropout_values[1]", TS(l.dropout_values[1])); line("      ", "dropout_values[2]", TS(0.f));
    };
    auto normalization = [&](size_t li) {   // Information__Layer__Normalization / __Normalized_Unit, :626-712
        const myea_layer_desc &l = desc_.layers[li];
        line("    ", "type_normalization", str(l.type_normalization));
        if (l.type_layer == MYEA_LAYER_FULLY_CONNECTED || l.type_layer == MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT)
            line("      ", "use_layer_normalization_before_activation", str(l.use_layer_normalization_before_activation));
        line("      ", "number_normalized_units", str(norm_units[li]));
        if (l.type_normalization == MYEA_NORMALIZATION_NONE) { for (size_t u = 0; u < norm_units[li]; ++u) { s += "        NormU["; s += str(u); s += "]\n"; } return; }
        for (size_t u = 0; u < norm_units[li]; ++u) {
            s += "        NormU["; s += str(u); s += "]\n";
            const bool held = total_norm != 0 && !mean[li].empty();
            // where unit u keeps its scale, and its statistics of step t.  An LSTM layer's units are written block by block, the
            // cell's three then the block's six (Neural_Network__Ordered.cpp:937-966), while their parameters and statistics are
            // held group by group; the [t] entries carry the group's own statistics of step t (the reference's writer steps through
            // them with the layer's unit count instead of the group's, Neural_Network__Save.cpp:695, so that for t > 0 its own file
            // does not hold what its forward pass used: nothing to follow there).
            size_t slot = u, stat0 = u, stat_stride = norm_units[li];
            if (l.type_layer == MYEA_LAYER_LSTM) {
                const size_t K = l.n_units, dir = u / (9 * K), k = (u % (9 * K)) / 9, g = u % 9;
                slot = dir * 9 * K + g * K + k; stat0 = (dir * 9 + g) * T * K + k; stat_stride = K;
            }
            line("          ", "scale", TS(held ? P[scale_at + l.first_normalized_unit_index + slot] : 1.f));
            line("          ", "shift", TS(held ? P[scale_at + total_norm + l.first_normalized_unit_index + slot] : 0.f));
            for (size_t t = 0; t < T; ++t) {
                line("          ", "mean_average[" + str(t) + "]", TS(held ? mean[li][t * stat_stride + stat0] : 0.f));
                line("          ", "variance_average[" + str(t) + "]", TS(held ? var[li][t * stat_stride + stat0] : 1.f));
            }
        }
    };
    // what a connection of layer `li` points at: ENUM_TYPE_LAYER_CONNECTION_NAME of its source layer and that layer's first unit
    auto source = [&](size_t li, const char **name, size_t *first) {
        const size_t pl = myea_net_desc_previous_layer(&desc_, (uint32_t)li);
        switch (desc_.layers[pl].type_layer) {
        case MYEA_LAYER_LSTM: *name = "connected_to_cell"; *first = cell_at[pl]; break;
        case MYEA_LAYER_RESIDUAL: case MYEA_LAYER_AVERAGE_POOLING: *name = "connected_to_basic"; *first = basic_at[pl]; break;
        case MYEA_LAYER_MAX_POOLING: *name = "connected_to_basic_indice"; *first = indice_at[pl]; break;
        default: *name = "connected_to_neuron"; *first = neuron_at[pl]; break;
        }
    };
    auto neurons = [&](size_t li, const char *count_key) {   // Information__Layer__FC / __Output_Layer, :714-824
        const myea_layer_desc &l = desc_.layers[li];
        const size_t H = width(li), In = width(myea_net_desc_previous_layer(&desc_, (uint32_t)li));
        const char *name; size_t first;
        source(li, &name, &first);
        line("    ", count_key, str(H));
        for (size_t o = 0; o < H; ++o) {
            s += "      Neuron_unit["; s += str(o); s += "]\n";
            line("        ", "number_connections", str(In));
            for (size_t k = 0; k < In; ++k) { line("          ", name, str(first + k)); weight("          ", l.first_connection_index + o * In + k); }
        }
    };
    auto af = [&](size_t li) {   // Information__Layer__AF, :826-842
        const myea_layer_desc &l = desc_.layers[li];
        line("    ", "number_AF_units", str(af_units[li]));
        for (size_t u = 0; u < af_units[li]; ++u) {
            s += "      AF["; s += str(u); s += "]\n";
            line("        ", "activation_steepness", TS(l.activation_steepness)); line("        ", "activation_function", str(l.type_activation_function));
        }
    };
    auto bias = [&](size_t first, size_t count) {   // Information__Layer__Bias, :865-879
        line("    ", "number_bias_parameters", str(count));
        for (size_t k = 0; k < count; ++k) weight("      ", first + k);
    };
    auto shared = [&](const myea_layer_desc &l) {
        line("    ", "use_tied_parameter", "0"); line("    ", "k_sparsity", str(l.k_sparsity)); line("    ", "alpha_sparsity", TS(l.k_sparsity ? l.alpha_sparsity : 1.f));
        line("    ", "constraint_recurrent_weight_lower_bound", TS(l.constraint_recurrent_weight_lower_bound));
        line("    ", "constraint_recurrent_weight_upper_bound", TS(l.constraint_recurrent_weight_upper_bound));
    };

    s += "  Input layer:\n";
    line("    ", "type_layer", str(desc_.layers[0].type_layer)); line("    ", "type_activation", "0");
    dropout(desc_.layers[0], false);
    line("    ", "number_inputs", str(width(0)));
    for (size_t li = 1; li + 1 < L; ++li) {
        const myea_layer_desc &l = desc_.layers[li];
        s += "  Hidden layer "; s += str(li); s += ":\n";
        line("    ", "type_layer", str(l.type_layer)); line("    ", "use_bidirectional", str(l.use_bidirectional));
        switch (l.type_layer) {
        case MYEA_LAYER_AVERAGE_POOLING: case MYEA_LAYER_MAX_POOLING:
            line("    ", "kernel_size", str(l.pooling_values[0])); line("    ", "stride", str(l.pooling_values[1])); line("    ", "padding", str(l.pooling_values[2]));
            line("    ", "dilation", str(l.pooling_values[3]));
            line("    ", l.type_layer == MYEA_LAYER_MAX_POOLING ? "number_basic_indice_units" : "number_basic_units", str(width(li)));
            break;
        case MYEA_LAYER_FULLY_CONNECTED: case MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT: {
            line("    ", "type_activation", str(io_detail::Class_Activation(l.type_activation_function)));
            dropout(l, true); normalization(li); shared(l);
            neurons(li, "number_neuron_units");
            if (l.type_layer == MYEA_LAYER_FULLY_CONNECTED) af(li);
            else {   // Information__Layer__AF_Ind_Recurrent, :844-863
                const size_t H = width(li), u0 = l.first_connection_index + H * width(myea_net_desc_previous_layer(&desc_, (uint32_t)li));
                line("    ", "number_AF_Ind_recurrent_units", str(af_units[li]));
                for (size_t u = 0; u < af_units[li]; ++u) {
                    s += "      AF_Ind_R["; s += str(u); s += "]\n";
                    line("        ", "activation_steepness", TS(l.activation_steepness)); line("        ", "activation_function", str(l.type_activation_function));
                    line("        ", "connected_to_AF_Ind_R", str(ind_at[li] + u)); weight("        ", u0 + u);
                }
            }
            bias(l.first_bias_connection_index, width(li));
            break;
        }
        case MYEA_LAYER_LSTM: {   // Information__Layer__LSTM / Layer__LSTM_Information__Connection, :899-1096
            const size_t K = l.n_units, cpb = l.n_cells_per_block, C = K * cpb, In = width(myea_net_desc_previous_layer(&desc_, (uint32_t)li)), D = dirs(li);
            const size_t per_block = cpb * (In + C) + 3 * In + 3 * C + 3 * cpb;
            const char *name; size_t first;
            source(li, &name, &first);
            line("    ", "type_activation", "5");   // symmetric (Prepare__Connections__LSTM, Neural_Network__Prepare_Connections.cpp:119)
            dropout(l, true); normalization(li); shared(l);
            line("    ", "number_block_units", str(K * D)); line("    ", "number_cell_units", str(C * D));
            for (size_t b = 0; b < K * D; ++b) {
                const size_t dir = b / K, cells0 = cell_at[li] + dir * C;   // the direction's own cells
                size_t at = l.first_connection_index + b * per_block;
                s += "      Block["; s += str(b); s += "]\n";
                line("        ", "activation_function", str(MYEA_AF_TANH)); s += "        activation_steepness 1\n";
                line("        ", "number_connections", str(per_block));
                auto forward = [&]() { for (size_t k = 0; k < In; ++k) { line("          ", name, str(first + k)); weight("          ", at++); } };
                auto recurrent = [&]() { for (size_t k = 0; k < C; ++k) { line("          ", "connected_to_cell", str(cells0 + k)); weight("          ", at++); } };
                for (size_t j = 0; j < cpb; ++j) { forward(); recurrent(); }   // cell inputs
                for (int g = 0; g < 3; ++g) forward();                         // input, forget, output gate
                for (int g = 0; g < 3; ++g) recurrent();
                for (int g = 0; g < 3; ++g)                                    // peepholes: the block's own cells
                    for (size_t k = 0; k < cpb; ++k) { line("          ", "connected_to_cell", str(cells0 + (b % K) * cpb + k)); weight("          ", at++); }
            }
            // Prepare__Bias__LSTM leaves [first, last) on the 3 x blocks gate biases (:232-250)
            bias(l.use_bidirectional ? l.first_bias_connection_index + C * D : l.first_bias_connection_index, 3 * K * D);
            break;
        }
        case MYEA_LAYER_RESIDUAL:
            line("    ", "block_depth", str(l.block_depth));
            {
                const size_t a = width(myea_net_desc_previous_layer(&desc_, (uint32_t)li)), b = width(li + l.block_depth);
                line("    ", "padding", str(((a > b ? a - b : b - a) + 1) / 2));
            }
            dropout(l, true); normalization(li);
            line("    ", "number_basic_units", str(width(li)));
            break;
        default: return Fail("Save_Dimension_Parameters", "layer type is not managed");
        }
    }
    {
        const size_t lo = L - 1;
        const myea_layer_desc &l = desc_.layers[lo];
        s += "  Output layer:\n";
        line("    ", "type_layer", str(l.type_layer)); line("    ", "type_activation", str(io_detail::Class_Activation(l.type_activation_function)));
        neurons(lo, "number_outputs"); af(lo); bias(l.first_bias_connection_index, width(lo));
    }
    s += "|END| DIMENSION |END|\n";
    std::ofstream f(path, std::ios::out | std::ios::binary);
    if (!f.is_open()) return Fail("Save_Dimension_Parameters", "the file can not be opened");
    f.write(s.c_str(), (std::streamsize)s.size());
    f.flush();
    return f.fail() ? Fail("Save_Dimension_Parameters", "write failed") : true;
}

inline bool Neural_Network_HIP::Load(std::string const &path_dimension, std::string const &path_parameters, size_t maximum_allowable_memory)
{
    (void)maximum_allowable_memory;
    io_detail::Tokens g, d;
    if (!g.Read(path_parameters)) return Fail("Load", "could not find the general parameters file");
    if (!d.Read(path_dimension)) return Fail("Load", "could not find the dimension parameters file");
    const char *fn = "Load";
    // ---- general parameters (Load_Parameters, Neural_Network__Load.cpp:82-2321), in the writer's order ----
    size_t u = 0;
    float skip = 0.f;
    bool ok = g.Real("learning_rate", &learning_rate) && g.Real("learning_rate_final", &learning_rate_final) && g.Real("learning_momentum", &learning_momentum) &&
              g.Real("learning_gamma", &learning_gamma) && g.Bool("use_Nesterov", &use_Nesterov) && g.Real("quickprop_decay", &skip) && g.Real("quickprop_mu", &skip) &&
              g.Real("rprop_increase_factor", &rprop_increase_factor) && g.Real("rprop_decrease_factor", &rprop_decrease_factor) && g.Real("rprop_delta_min", &rprop_delta_min) &&
              g.Real("rprop_delta_max", &rprop_delta_max) && g.Real("rprop_delta_zero", &rprop_delta_zero) && g.Real("sarprop_epoch", &skip) &&
              g.Real("adam_learning_rate", &adam_learning_rate) && g.Real("adam_beta1", &adam_beta1) && g.Real("adam_beta2", &adam_beta2) && g.Real("adam_epsilon", &adam_epsilon) &&
              g.Bool("adam_bias_correction", &use_adam_bias_correction) && g.Real("adam_gamma", &adam_gamma) && g.Bool("use_Warm_Restarts", &use_Warm_Restarts) &&
              g.Real("warm_restarts_decay_learning_rate", &warm_restarts_decay_learning_rate) && g.Real("warm_restarts_maximum_learning_rate", &warm_restarts_initial_maximum_learning_rate) &&
              g.Real("warm_restarts_minimum_learning_rate", &warm_restarts_minimum_learning_rate) && g.Real("warm_restarts_initial_T_i", &warm_restarts_initial_T_i) &&
              g.Real("warm_restarts_multiplier", &warm_restarts_multiplier);
    if (!ok) return Fail(fn, "general parameters: a field of the optimizer sections is missing");
    warm_restarts_maximum_learning_rate = warm_restarts_initial_maximum_learning_rate; warm_restarts_T_i = warm_restarts_initial_T_i;
    ok = g.Size("type_optimizer_function", &u); type_optimizer_function = (unsigned)u;
    ok = ok && g.Size("type_loss_function", &u); type_loss_function = (unsigned)u;
    ok = ok && g.Size("type_accuracy_function", &u); type_accuracy_function = (unsigned)u;
    ok = ok && g.Real("bit_fail_limit", &bit_fail_limit) && g.Size("pre_training_level", &u) && g.Bool("use_clip_gradient", &use_clip_gradient) && g.Real("clip_gradient", &clip_gradient) &&
         g.Real("regularization__max_norm_constraints", &regularization__max_norm_constraints) && g.Real("regularization__weight_decay", &regularization__weight_decay) &&
         g.Bool("use_normalized_weight_decay", &use_normalized_weight_decay) && g.Real("normalization_momentum_average", &normalization_momentum_average) &&
         g.Real("normalization_epsilon", &normalization_epsilon) && g.Real("batch_renormalization_r_correction_maximum", &batch_renormalization_r_correction_maximum) &&
         g.Real("batch_renormalization_d_correction_maximum", &batch_renormalization_d_correction_maximum) && g.Real("loss_training", &loss_training) &&
         g.Real("loss_validating", &loss_validating) && g.Real("loss_testing", &loss_testing) && g.Real("accuracy_variance", &accuracy_variance) &&
         g.Real("accuracy_training", &accuracy_training) && g.Real("accuracy_validating", &accuracy_validating) && g.Real("accuracy_testing", &accuracy_testing);
    if (!ok) return Fail(fn, "general parameters: a field of the training sections is missing");

    // ---- dimension parameters (Load, :2323-6882) ----
    size_t type_network = 0, L = 0, T = 0, delays = 0, total_parameters_file = 0;
    if (!d.Size("type_network", &type_network) || !d.Size("number_layers", &L) || !d.Size("number_recurrent_depth", &T) || !d.Size("number_time_delays", &delays) ||
        !d.Size("total_parameters", &total_parameters_file))
        return Fail(fn, "dimension parameters: header incomplete");
    if (L < 2 || L > MYEA_MAX_LAYERS || T == 0) return Fail(fn, "dimension parameters: layer count or recurrent depth out of range");
    Deallocate();
    std::memset(&desc_, 0, sizeof(desc_));
    desc_.type_network = (uint32_t)type_network; desc_.n_layers = (uint32_t)L; desc_.number_recurrent_depth = (uint32_t)T; desc_.batch_size = (uint32_t)batch_size;
    number_recurrent_depth = T; number_time_delays = delays;
    struct Pending { size_t index; float value; };
    std::vector<Pending> weights;
    weights.reserve(total_parameters_file);
    struct NormRead { std::vector<float> scale, shift, mean, var; };
    std::vector<NormRead> norms(L);
    auto read_dropout = [&](myea_layer_desc &l, bool hidden) {
        size_t type = 0; bool coded = false;
        if (!d.Size("type_dropout", &type)) return false;
        if (hidden && !d.Bool("use_coded_dropout", &coded)) return false;
        l.type_dropout = (uint32_t)type;
        float unused;
        if (!d.Real("dropout_values[0]", &l.dropout_values[0]) || !d.Real("dropout_values[1]", &l.dropout_values[1]) || !d.Real("dropout_values[2]", &unused)) return false;
        if (type == MYEA_DROPOUT_GAUSSIAN) l.dropout_values[0] = l.dropout_values[0] == 1.f ? 0.f : (float)((double)l.dropout_values[0] / (1.0 - (double)l.dropout_values[0]));
        if (type == MYEA_DROPOUT_NONE) { l.dropout_values[0] = 1.f; l.dropout_values[1] = 0.f; }
        return true;
    };
    auto read_normalization = [&](size_t li, bool dense) {
        myea_layer_desc &l = desc_.layers[li];
        size_t type = 0, units = 0; bool before = true;
        if (!d.Size("type_normalization", &type)) return false;
        if (dense && !d.Bool("use_layer_normalization_before_activation", &before)) return false;
        if (!d.Size("number_normalized_units", &units)) return false;
        l.type_normalization = (uint32_t)type; l.use_layer_normalization_before_activation = before;
        if (type == MYEA_NORMALIZATION_NONE) return true;
        NormRead &n = norms[li];
        n.scale.resize(units); n.shift.resize(units); n.mean.resize(T * units); n.var.resize(T * units);
        for (size_t k = 0; k < units; ++k) {
            if (!d.Real("scale", &n.scale[k]) || !d.Real("shift", &n.shift[k])) return false;
            for (size_t t = 0; t < T; ++t) {
                const std::string mk = "mean_average[" + std::to_string(t) + "]", vk = "variance_average[" + std::to_string(t) + "]";
                if (!d.Real(mk.c_str(), &n.mean[t * units + k]) || !d.Real(vk.c_str(), &n.var[t * units + k])) return false;
            }
        }
        return true;
    };
    auto read_shared = [&](myea_layer_desc &l) {
        size_t k = 0; bool tied = false;
        if (!d.Bool("use_tied_parameter", &tied) || !d.Size("k_sparsity", &k) || !d.Real("alpha_sparsity", &l.alpha_sparsity) ||
            !d.Real("constraint_recurrent_weight_lower_bound", &l.constraint_recurrent_weight_lower_bound) ||
            !d.Real("constraint_recurrent_weight_upper_bound", &l.constraint_recurrent_weight_upper_bound)) return false;
        l.k_sparsity = (uint32_t)k;
        return !tied;   // tied parameters are not on this path
    };
    auto read_weights = [&](size_t count) {
        for (size_t k = 0; k < count; ++k) { Pending p; if (!d.Weight(&p.index, &p.value)) return false; weights.push_back(p); }
        return true;
    };
    auto read_neurons = [&](const char *count_key, size_t *units) {
        if (!d.Size(count_key, units)) return false;
        for (size_t o = 0; o < *units; ++o) { size_t c = 0; if (!d.Size("number_connections", &c) || !read_weights(c)) return false; }
        return true;
    };
    auto read_af = [&](myea_layer_desc &l, const char *count_key, bool recurrent, size_t class_read) {
        size_t units = 0;
        if (!d.Size(count_key, &units)) return false;
        if (units == 0) {   // the first layer of a residual block owns no activation unit: only the class is in the file
            static const uint32_t of_class[6] = {MYEA_AF_NONE, MYEA_AF_SIGMOID, MYEA_AF_RELU, MYEA_AF_SELU, MYEA_AF_SOFTMAX, MYEA_AF_TANH};
            l.type_activation_function = class_read < 6 ? of_class[class_read] : MYEA_AF_SIGMOID;
            if (l.type_activation_function == MYEA_AF_NONE) l.type_activation_function = MYEA_AF_SIGMOID;
        }
        for (size_t k = 0; k < units; ++k) {
            float steep = 1.f; size_t f = 0;
            if (!d.Real("activation_steepness", &steep) || !d.Size("activation_function", &f)) return false;
            if (k == 0) { l.activation_steepness = steep; l.type_activation_function = (uint32_t)f; }
            else if (steep != l.activation_steepness || f != l.type_activation_function) return false;   // per-unit functions: set them through the C ABI
            if (recurrent && !read_weights(1)) return false;
        }
        return true;
    };
    auto read_bias = [&]() { size_t c = 0; return d.Size("number_bias_parameters", &c) && read_weights(c); };

    {   // input layer
        myea_layer_desc &l = desc_.layers[0];
        size_t type = 0, inputs = 0;
        if (!d.Skip("Input") || !d.Size("type_layer", &type) || !read_dropout(l, false) || !d.Size("number_inputs", &inputs)) return Fail(fn, "dimension parameters: input layer");
        l.type_layer = (uint32_t)type; l.n_units = (uint32_t)inputs; l.activation_steepness = 1.f; l.use_layer_normalization_before_activation = 1; l.alpha_sparsity = 1.f;
    }
    for (size_t li = 1; li + 1 < L; ++li) {
        myea_layer_desc &l = desc_.layers[li];
        size_t type = 0, v = 0; bool bidirectional = false;
        if (!d.Skip("Hidden") || !d.Size("type_layer", &type) || !d.Bool("use_bidirectional", &bidirectional)) return Fail(fn, "dimension parameters: hidden layer header");
        l.type_layer = (uint32_t)type; l.use_bidirectional = bidirectional; l.activation_steepness = 1.f; l.use_layer_normalization_before_activation = 1;
        l.dropout_values[0] = 1.f; l.alpha_sparsity = 1.f;
        switch (type) {
        case MYEA_LAYER_AVERAGE_POOLING: case MYEA_LAYER_MAX_POOLING: {
            size_t k = 0, st = 0, pad = 0, dil = 0, units = 0;
            if (!d.Size("kernel_size", &k) || !d.Size("stride", &st) || !d.Size("padding", &pad) || !d.Size("dilation", &dil) ||
                !d.Size(type == MYEA_LAYER_MAX_POOLING ? "number_basic_indice_units" : "number_basic_units", &units)) return Fail(fn, "dimension parameters: pooling layer");
            l.pooling_values[0] = (uint32_t)k; l.pooling_values[1] = (uint32_t)st; l.pooling_values[2] = (uint32_t)pad; l.pooling_values[3] = (uint32_t)dil;
            l.n_units = (uint32_t)units;   // the ceil mode is not in the file: chosen below so that the width comes out as written
            break;
        }
        case MYEA_LAYER_FULLY_CONNECTED: case MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT: {
            size_t units = 0;
            if (!d.Size("type_activation", &v) || !read_dropout(l, true) || !read_normalization(li, true) || !read_shared(l) || !read_neurons("number_neuron_units", &units))
                return Fail(fn, "dimension parameters: fully-connected layer");
            l.n_units = (uint32_t)units;
            if (!read_af(l, type == MYEA_LAYER_FULLY_CONNECTED ? "number_AF_units" : "number_AF_Ind_recurrent_units", type != MYEA_LAYER_FULLY_CONNECTED, v) || !read_bias())
                return Fail(fn, "dimension parameters: activation units or bias of a fully-connected layer (per-unit activation functions are set through the C ABI)");
            break;
        }
        case MYEA_LAYER_LSTM: {
            size_t blocks = 0, cells = 0;
            if (!d.Size("type_activation", &v) || !read_dropout(l, true) || !read_normalization(li, false) || !read_shared(l) || !d.Size("number_block_units", &blocks) ||
                !d.Size("number_cell_units", &cells) || blocks == 0) return Fail(fn, "dimension parameters: LSTM layer");
            const size_t D = bidirectional ? 2 : 1;
            l.n_units = (uint32_t)(blocks / D); l.n_cells_per_block = (uint32_t)(cells / blocks);
            for (size_t b = 0; b < blocks; ++b) { size_t c = 0; if (!d.Size("number_connections", &c) || !read_weights(c)) return Fail(fn, "dimension parameters: LSTM block"); }
            if (!read_bias()) return Fail(fn, "dimension parameters: LSTM bias");
            break;
        }
        case MYEA_LAYER_RESIDUAL: {
            size_t depth = 0, pad = 0, units = 0;
            if (!d.Size("block_depth", &depth) || !d.Size("padding", &pad) || !read_dropout(l, true) || !read_normalization(li, false) || !d.Size("number_basic_units", &units))
                return Fail(fn, "dimension parameters: residual layer");
            l.block_depth = (uint32_t)depth;
            break;
        }
        default: return Fail(fn, "dimension parameters: layer type is not on this path");
        }
    }
    {   // output layer
        myea_layer_desc &l = desc_.layers[L - 1];
        size_t type = 0, v = 0, units = 0;
        if (!d.Skip("Output") || !d.Size("type_layer", &type) || !d.Size("type_activation", &v) || !read_neurons("number_outputs", &units) || !read_af(l, "number_AF_units", false, v) || !read_bias())
            return Fail(fn, "dimension parameters: output layer");
        l.type_layer = (uint32_t)type; l.n_units = (uint32_t)units; l.use_layer_normalization_before_activation = 1; l.dropout_values[0] = 1.f; l.alpha_sparsity = 1.f;
    }
    // pooling widths: floor mode first, ceil mode when that is what reproduces the written width
    std::vector<uint32_t> written(L, 0);
    for (size_t li = 1; li + 1 < L; ++li) written[li] = desc_.layers[li].n_units;
    if (!Relayout(fn)) return false;
    for (size_t li = 1; li + 1 < L; ++li) {
        myea_layer_desc &l = desc_.layers[li];
        if ((l.type_layer != MYEA_LAYER_AVERAGE_POOLING && l.type_layer != MYEA_LAYER_MAX_POOLING) || l.n_units == written[li]) continue;
        l.pooling_values[4] = 1;
        if (!Relayout(fn)) return false;
        if (desc_.layers[li].n_units != written[li]) return Fail(fn, "dimension parameters: a pooling layer's width does not follow from its parameters");
    }
    if (desc_.total_parameters != total_parameters_file) return Fail(fn, "dimension parameters: total_parameters does not match the layers");
    for (const Pending &p : weights) {
        if (p.index >= desc_.total_weights + desc_.total_bias) return Fail(fn, "dimension parameters: weight index overflow");
        ptr_array_parameters[p.index] = p.value;
    }
    norm_means_averages_.assign(L, std::vector<float>()); norm_variances_averages_.assign(L, std::vector<float>());
    for (size_t li = 0; li < L; ++li) {
        const NormRead &n = norms[li];
        if (n.scale.empty()) continue;
        const myea_layer_desc &l = desc_.layers[li];
        const size_t at = desc_.total_weights + desc_.total_bias + l.first_normalized_unit_index;
        if (desc_.total_normalized_units == 0 || l.first_normalized_unit_index + n.scale.size() > desc_.total_normalized_units) return Fail(fn, "dimension parameters: normalised units overflow");
        if (l.type_layer == MYEA_LAYER_LSTM) {   // units written block by block, held group by group: see the writer
            if (l.n_cells_per_block != 1) return Fail(fn, "dimension parameters: a normalised LSTM layer needs one cell per block");
            const size_t K = l.n_units, units = n.scale.size();
            norm_means_averages_[li].assign(T * units, 0.f); norm_variances_averages_[li].assign(T * units, 1.f);
            for (size_t u = 0; u < units; ++u) {
                const size_t dir = u / (9 * K), k = (u % (9 * K)) / 9, g = u % 9, slot = dir * 9 * K + g * K + k;
                ptr_array_parameters[at + slot] = n.scale[u]; ptr_array_parameters[at + desc_.total_normalized_units + slot] = n.shift[u];
                for (size_t t = 0; t < T; ++t) {
                    norm_means_averages_[li][((dir * 9 + g) * T + t) * K + k] = n.mean[t * units + u];
                    norm_variances_averages_[li][((dir * 9 + g) * T + t) * K + k] = n.var[t * units + u];
                }
            }
            continue;
        }
        for (size_t k = 0; k < n.scale.size(); ++k) { ptr_array_parameters[at + k] = n.scale[k]; ptr_array_parameters[at + desc_.total_normalized_units + k] = n.shift[k]; }
        norm_means_averages_[li] = n.mean; norm_variances_averages_[li] = n.var;
    }
    return true;
}

}  // namespace MyEA_HIP
