/* myea_layout.c — host-side descriptor logic of the C ABI (no GPU code).
 *
 * Reproduces the index assignment of `Neural_Network::Compile` so that callers without a host
 * `Neural_Network` object (tests, the benchmark, the C++ adaptor) address the flat parameter vector
 * exactly as the reference does.  NN/ = Neural_Network_Library_Windows/Source_Files/Neural_Network/.
 */
#include "../../include/myea_hip.h"

#include <float.h>
#include <math.h>
#include <string.h>

/* Public training fields: Header_Files/Neural_Network/Data.hpp:2929-2970. */
void myea_hyper_default(myea_hyper *h)
{
    if (!h) return;
    memset(h, 0, sizeof(*h));
    h->type_optimizer_function = MYEA_OPTIMIZER_NONE;
    h->type_loss_function = MYEA_LOSS_NONE;
    h->type_accuracy_function = MYEA_ACCURACY_DISTANCE;
    h->use_Nesterov = 0;
    h->use_adam_bias_correction = 1;
    h->use_clip_gradient = 0;
    h->learning_rate = 0.01f;
    h->learning_rate_final = 0.1f;
    h->learning_momentum = 0.9f;
    h->learning_gamma = 1e-3f;
    h->adam_learning_rate = 0.001f;
    h->adam_beta1 = 0.9f;
    h->adam_beta2 = 0.999f;
    h->adam_epsilon = 1e-8f;
    h->regularization__weight_decay = 0.f;
    h->clip_gradient = 1.f;
    h->accuracy_variance = 0.49f;
    h->bit_fail_limit = 0.35f;
    h->normalization_momentum_average = 0.999f;
    h->normalization_epsilon = 1e-5f;
    h->batch_renormalization_r_correction_maximum = 1.f;
    h->batch_renormalization_d_correction_maximum = 0.f;
    h->optimizer_time_step = 0.f;
    h->number_time_delays = 0;
    h->use_normalized_weight_decay = 1;
    h->epoch_time_step = 1.f;
    h->adam_gamma = 0.1f;
    h->adam_previous_beta2 = 0.f;
    h->rprop_increase_factor = 1.2f;
    h->rprop_decrease_factor = 0.5f;
    h->rprop_delta_min = 1e-6f;
    h->rprop_delta_max = 50.f;
    h->rprop_delta_zero = 0.1f;
    h->loss_rprop = FLT_MAX;
    h->previous_loss_rprop = FLT_MAX;
    h->regularization__max_norm_constraints = 0.f;
    h->use_Warm_Restarts = 0;
    h->warm_restarts_decay_learning_rate = 1.f;
    h->warm_restarts_maximum_learning_rate = 1.f;
    h->warm_restarts_minimum_learning_rate = 1e-7f;
    h->warm_restarts_T_i = 1.f;
    h->warm_restarts_multiplier = 2.f;
}

/* Index of the residual layer whose block contains layer li, or 0 when li is outside every block
 * (layer 0 is the input layer and never a residual layer).  Blocks do not nest here. */
static uint32_t enclosing_block(const myea_net_desc *d, uint32_t li)
{
    for (uint32_t r = 1; r < li; ++r) {
        const myea_layer_desc *l = &d->layers[r];
        if (l->type_layer == MYEA_LAYER_RESIDUAL && li <= r + l->block_depth) return r;
    }
    return 0;
}

/* previous_connected_layers[0] (Organize__Previous_Layers_Connected, NN/Neural_Network.cpp:20-57): the layer
 * before; the first layer after a residual block connects to the block's residual layer; the first layer inside a
 * block connects to what the residual layer itself connects to (the shortcut source). */
uint32_t myea_net_desc_previous_layer(const myea_net_desc *d, uint32_t li)
{
    if (!d || li == 0 || li >= d->n_layers) return 0;
    uint32_t before = li - 1;
    if (d->layers[before].type_layer == MYEA_LAYER_RESIDUAL) return myea_net_desc_previous_layer(d, before);
    uint32_t r = enclosing_block(d, before);
    if (r != 0 && before == r + d->layers[r].block_depth && enclosing_block(d, li) != r) return r;
    return before;
}

/* *Layer::ptr_number_outputs: FC = neurons; LSTM = blocks * cells per direction
 * (NN/Neural_Network__Compile.cpp:79); residual = the wider of the shortcut source and the block's last layer
 * (Assign__Post__Layer, NN/Neural_Network__Compile.cpp:272-281). */
uint64_t myea_net_desc_number_outputs(const myea_net_desc *d, uint32_t li)
{
    if (!d || li >= d->n_layers) return 0;
    const myea_layer_desc *l = &d->layers[li];
    switch (l->type_layer) {
    case MYEA_LAYER_LSTM: return (uint64_t)l->n_units * l->n_cells_per_block;
    case MYEA_LAYER_RESIDUAL: {
        uint64_t a = myea_net_desc_number_outputs(d, myea_net_desc_previous_layer(d, li));
        uint64_t b = myea_net_desc_number_outputs(d, li + l->block_depth);
        return a > b ? a : b;
    }
    default: return l->n_units;
    }
}
#define number_outputs myea_net_desc_number_outputs
#define previous_layer myea_net_desc_previous_layer

static int is_pooling(const myea_layer_desc *l) { return l->type_layer == MYEA_LAYER_AVERAGE_POOLING || l->type_layer == MYEA_LAYER_MAX_POOLING; }
static int is_ind_rnn(const myea_layer_desc *l) { return l->type_layer == MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT; }
/* neuron units + activation units: fully-connected and independently recurrent layers */
static int is_dense(const myea_layer_desc *l) { return l->type_layer == MYEA_LAYER_FULLY_CONNECTED || is_ind_rnn(l); }

int myea_net_desc_layout(myea_net_desc *d)
{
    if (!d || d->n_layers < 2 || d->n_layers > MYEA_MAX_LAYERS) return MYEA_E_INVALID;
    if (d->number_recurrent_depth == 0 || d->batch_size == 0) return MYEA_E_INVALID;
    uint64_t total_weights = 0, total_bias = 0;
    int any_norm = 0;

    for (uint32_t li = 0; li < d->n_layers; ++li) {
        myea_layer_desc *l = &d->layers[li];
        const int pooling = is_pooling(l);
        if (l->n_units == 0 && l->type_layer != MYEA_LAYER_RESIDUAL && !pooling) return MYEA_E_INVALID;
        if (l->type_layer == MYEA_LAYER_LSTM && l->n_cells_per_block == 0) return MYEA_E_INVALID;
        if (!is_dense(l) && l->type_layer != MYEA_LAYER_LSTM && l->type_layer != MYEA_LAYER_RESIDUAL && !pooling) return MYEA_E_UNSUPPORTED;
        if (is_ind_rnn(l) && (li == 0 || li + 1 == d->n_layers)) return MYEA_E_INVALID;
        if (l->k_sparsity != 0) {
            /* Set__K_Sparsity / Set__Alpha_Sparsity (NN/Neural_Network__K_Sparse.cpp:38-190): hidden layers, alpha >= 0,
             * size_t(k * alpha) <= width.  Here also k <= width and at least one value kept at inference (the reference
             * reads its pair array's first slot whatever k is). */
            const float scaled = (float)l->k_sparsity * l->alpha_sparsity;
            if (li == 0 || li + 1 == d->n_layers || l->type_layer != MYEA_LAYER_FULLY_CONNECTED) return MYEA_E_UNSUPPORTED;
            if (l->k_sparsity > l->n_units || !(l->alpha_sparsity >= 0.f) || !(scaled >= 1.f) || (uint64_t)scaled > l->n_units) return MYEA_E_INVALID;
        }
        if (pooling && (l->pooling_values[0] == 0 || l->pooling_values[1] == 0 || li == 0 || li + 1 == d->n_layers)) return MYEA_E_INVALID;
        if (l->type_normalization != MYEA_NORMALIZATION_NONE) any_norm = 1;
    }
    if (d->layers[0].type_layer != MYEA_LAYER_FULLY_CONNECTED || d->layers[d->n_layers - 1].type_layer != MYEA_LAYER_FULLY_CONNECTED) return MYEA_E_INVALID;
    /* widths of the pooling layers, in layer order (Assign__Post__Layer, NN/Neural_Network__Compile.cpp:250-271):
     * average: floor or ceil((In + 2 padding - kernel) / stride + 1) - the dilation is not in the formula;
     * max:     floor or ceil((In + 2 padding - dilation (kernel - 1) - 1) / stride + 1) */
    for (uint32_t li = 1; li < d->n_layers; ++li) {
        myea_layer_desc *l = &d->layers[li];
        if (!is_pooling(l)) continue;
        /* inside a residual block too (Assign__Post__Residual_Layer, NN/Neural_Network__Compile.cpp:352-376, computes a member's
         * width by the same formulas) */
        const double in = (double)number_outputs(d, previous_layer(d, li));
        const double kernel = l->pooling_values[0], stride = l->pooling_values[1], padding = l->pooling_values[2], dilation = l->pooling_values[3];
        const double span = l->type_layer == MYEA_LAYER_AVERAGE_POOLING ? in + 2.0 * padding - kernel : in + 2.0 * padding - dilation * (kernel - 1.0) - 1.0;
        if (span < 0.0) return MYEA_E_INVALID;
        const double out = l->pooling_values[4] == 0 ? floor(span / stride + 1.0) : ceil(span / stride + 1.0);
        if (out < 1.0 || out > 4294967295.0) return MYEA_E_INVALID;
        l->n_units = (uint32_t)out;
    }
    /* residual blocks: depth >= 1, wholly inside the stack, followed by at least one layer; fully-connected, independently
     * recurrent, LSTM and pooling members (what Recurrent__Forward_Pass__Residual__Layer's switch knows,
     * NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:711-771), no block inside a block */
    for (uint32_t li = 1; li < d->n_layers; ++li) {
        const myea_layer_desc *l = &d->layers[li];
        if (l->type_layer != MYEA_LAYER_RESIDUAL) continue;
        if (l->block_depth == 0 || (uint64_t)li + l->block_depth + 1 >= d->n_layers) return MYEA_E_INVALID;
        for (uint32_t k = 1; k <= l->block_depth; ++k)
            if (d->layers[li + k].type_layer == MYEA_LAYER_RESIDUAL) return MYEA_E_UNSUPPORTED;
        li += l->block_depth;
    }

    /* weights: Prepare__Connections__FC / __FC_Ind_RNN / __LSTM, NN/Neural_Network__Prepare_Connections.cpp:20-222.
     * An independently recurrent layer's self weights (one per unit) follow its [units][fan-in] matrix (:45-77). */
    for (uint32_t li = 1; li < d->n_layers; ++li) {
        myea_layer_desc *l = &d->layers[li];
        if (l->type_layer == MYEA_LAYER_RESIDUAL || is_pooling(l)) { l->first_connection_index = l->last_connection_index = total_weights; continue; }
        uint64_t fan_in = number_outputs(d, previous_layer(d, li));
        l->first_connection_index = total_weights;
        if (is_dense(l)) {
            /* one self weight per recurrent activation unit: as many as the layer has units; inside a residual block they sit on
             * the layer's input side - fan-in many, none for the block's first layer (Assign__Post__Residual_Layer,
             * NN/Neural_Network__Compile.cpp:385-392) */
            const uint32_t r = enclosing_block(d, li);
            const uint64_t recurrent_units = !is_ind_rnn(l) ? 0u : (r == 0 ? l->n_units : (li == r + 1 ? 0u : fan_in));
            total_weights += fan_in * l->n_units + recurrent_units;
        } else { /* LSTM */
            uint64_t dirs = l->use_bidirectional ? 2u : 1u;
            uint64_t cpb = l->n_cells_per_block, cells_per_layer = (uint64_t)l->n_units * cpb;
            uint64_t per_block = cpb * (fan_in + cells_per_layer) + 3u * fan_in + 3u * cells_per_layer + 3u * cpb;
            total_weights += per_block * l->n_units * dirs;
        }
        l->last_connection_index = total_weights;
    }
    /* biases: Prepare__Bias__FC / __LSTM, :224-252.  The LSTM variant leaves first_bias_connection_index
     * pointing one cell-count past the start of the layer's slice (the second assignment at :246
     * overwrites the first at :240); the kernels use the field as stored. */
    for (uint32_t li = 1; li < d->n_layers; ++li) {
        myea_layer_desc *l = &d->layers[li];
        if (l->type_layer == MYEA_LAYER_RESIDUAL || is_pooling(l)) { l->first_bias_connection_index = total_weights + total_bias; continue; }
        if (is_dense(l)) {
            l->first_bias_connection_index = total_weights + total_bias;
            total_bias += l->n_units;
        } else {
            uint64_t dirs = l->use_bidirectional ? 2u : 1u;
            uint64_t cells = (uint64_t)l->n_units * l->n_cells_per_block * dirs, blocks = (uint64_t)l->n_units * dirs;
            /* one direction: the field as the reference leaves it.  Two directions: the reference splits
             * [first, last) in halves before either is assigned (Allocate__Bidirectional__Layers runs ahead of
             * Prepare__Bias__LSTM, NN/Neural_Network__Compile.cpp:542 vs :665) and overlays the directions' buffers, so
             * there is no working behaviour to follow; here direction d owns the contiguous [z | i | f | o] vectors at
             * first_bias_connection_index + d * (cells + 3 * blocks) per direction, starting at the slice's start. */
            l->first_bias_connection_index = total_weights + total_bias + (l->use_bidirectional ? 0u : cells);
            total_bias += cells + 3u * blocks;
        }
    }
    d->layers[0].first_connection_index = d->layers[0].last_connection_index = 0;
    d->layers[0].first_bias_connection_index = 0;

    /* normalised units: every layer owns Normalized_unit entries whether or not it is normalised
     * (Prepare__Normalized__Layers, NN/Neural_Network__Layer_Normalization.cpp:20-78); the scale / shift
     * region exists once any layer is normalised (Allocate__Parameter__Normalization,
     * NN/Neural_Network__Allocate.cpp:2378-2406). */
    uint64_t total_norm = 0;
    for (uint32_t li = 0; li < d->n_layers; ++li) {
        myea_layer_desc *l = &d->layers[li];
        l->first_normalized_unit_index = total_norm;
        if (l->type_layer == MYEA_LAYER_LSTM) {
            uint64_t dirs = l->use_bidirectional ? 2u : 1u;
            total_norm += 3u * (uint64_t)l->n_units * l->n_cells_per_block * dirs + 6u * (uint64_t)l->n_units * dirs;
        } else if (is_pooling(l)) {
            /* pooling layers own none (Prepare__Normalized__Layer, NN/Neural_Network__Layer_Normalization.cpp:44-45) */
        } else if (l->type_layer == MYEA_LAYER_RESIDUAL) {
            total_norm += number_outputs(d, li + l->block_depth);   /* Prepare__Normalized__Layer, :60-67 */
        } else if (enclosing_block(d, li) != 0) {
            total_norm += number_outputs(d, previous_layer(d, li)); /* Prepare__Normalized__Residual_Layer: fan-in wide */
        } else {
            total_norm += number_outputs(d, li);
        }
    }
    /* Bernoulli masks: (AF units of the layer) * T per layer, in layer order
     * (Reset__Parameter__Mask_Dropout, NN/Neural_Network.cpp:3948-3962); LSTM and residual layers own no AF unit. */
    uint64_t total_mask = 0;
    for (uint32_t li = 0; li < d->n_layers; ++li) {
        myea_layer_desc *l = &d->layers[li];
        l->first_mask_index = total_mask;
        if (!is_dense(l)) continue;   /* AF_unit and AF_Ind_recurrent_unit alike, :3959-3960 */
        uint32_t r = li ? enclosing_block(d, li) : 0;
        /* inside a block the activation units sit on the layer's input side: none for the block's first layer, fan-in
         * many for the others (Assign__Post__Residual_Layer, NN/Neural_Network__Compile.cpp:378-384) */
        uint64_t af_units = r == 0 ? l->n_units : (li == r + 1 ? 0 : number_outputs(d, previous_layer(d, li)));
        total_mask += af_units * d->number_recurrent_depth;
    }
    d->total_weights = total_weights;
    d->total_bias = total_bias;
    d->total_normalized_units = any_norm ? total_norm : 0;
    d->total_parameters = total_weights + total_bias + 2u * d->total_normalized_units;
    d->total_mask_units = total_mask;
    return MYEA_OK;
}
