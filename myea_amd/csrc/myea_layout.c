/* myea_layout.c — host-side descriptor logic of the C ABI (no GPU code).
 *
 * Reproduces the index assignment of `Neural_Network::Compile` so that callers without a host
 * `Neural_Network` object (tests, the benchmark, the C++ adaptor) address the flat parameter vector
 * exactly as the reference does.  NN/ = Neural_Network_Library_Windows/Source_Files/Neural_Network/.
 */
#include "../../include/myea_hip.h"

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
}

/* *Layer::ptr_number_outputs: FC = neurons; LSTM = blocks * cells per direction
 * (NN/Neural_Network__Compile.cpp:79); residual = width of the block's last layer. */
static uint64_t number_outputs(const myea_net_desc *d, uint32_t li)
{
    const myea_layer_desc *l = &d->layers[li];
    switch (l->type_layer) {
    case MYEA_LAYER_LSTM: return (uint64_t)l->n_units * l->n_cells_per_block;
    case MYEA_LAYER_RESIDUAL: return number_outputs(d, li + l->block_depth);
    default: return l->n_units;
    }
}

/* previous_connected_layers[0] for a sequential stack: the layer before, except that the first layer
 * after a residual block connects to the block's unit (NN/Neural_Network__Ordered.cpp, Order__Layers__Connection). */
static uint32_t previous_layer(const myea_net_desc *d, uint32_t li)
{
    /* walk back: if li-1 is the last layer inside a residual block, the producer is that block's layer */
    for (uint32_t r = 0; r + 1 < li; ++r) {
        const myea_layer_desc *l = &d->layers[r];
        if (l->type_layer == MYEA_LAYER_RESIDUAL && r + l->block_depth == li - 1) return r;
    }
    return li - 1;
}

int myea_net_desc_layout(myea_net_desc *d)
{
    if (!d || d->n_layers < 2 || d->n_layers > MYEA_MAX_LAYERS) return MYEA_E_INVALID;
    if (d->number_recurrent_depth == 0 || d->batch_size == 0) return MYEA_E_INVALID;
    uint64_t total_weights = 0, total_bias = 0;
    int any_norm = 0;

    for (uint32_t li = 0; li < d->n_layers; ++li) {
        myea_layer_desc *l = &d->layers[li];
        if (l->n_units == 0 && l->type_layer != MYEA_LAYER_RESIDUAL) return MYEA_E_INVALID;
        if (l->type_layer == MYEA_LAYER_LSTM && l->n_cells_per_block == 0) return MYEA_E_INVALID;
        if (l->type_layer != MYEA_LAYER_FULLY_CONNECTED && l->type_layer != MYEA_LAYER_LSTM &&
            l->type_layer != MYEA_LAYER_RESIDUAL) return MYEA_E_UNSUPPORTED;
        if (l->type_normalization != MYEA_NORMALIZATION_NONE) any_norm = 1;
    }
    if (d->layers[0].type_layer != MYEA_LAYER_FULLY_CONNECTED) return MYEA_E_INVALID;

    /* weights: Prepare__Connections__FC / __LSTM, NN/Neural_Network__Prepare_Connections.cpp:20-222 */
    for (uint32_t li = 1; li < d->n_layers; ++li) {
        myea_layer_desc *l = &d->layers[li];
        if (l->type_layer == MYEA_LAYER_RESIDUAL) { l->first_connection_index = l->last_connection_index = total_weights; continue; }
        uint64_t fan_in = number_outputs(d, previous_layer(d, li));
        l->first_connection_index = total_weights;
        if (l->type_layer == MYEA_LAYER_FULLY_CONNECTED) {
            total_weights += fan_in * l->n_units;
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
        if (l->type_layer == MYEA_LAYER_RESIDUAL) { l->first_bias_connection_index = total_weights + total_bias; continue; }
        if (l->type_layer == MYEA_LAYER_FULLY_CONNECTED) {
            l->first_bias_connection_index = total_weights + total_bias;
            total_bias += l->n_units;
        } else {
            uint64_t dirs = l->use_bidirectional ? 2u : 1u;
            uint64_t cells = (uint64_t)l->n_units * l->n_cells_per_block * dirs, blocks = (uint64_t)l->n_units * dirs;
            l->first_bias_connection_index = total_weights + total_bias + cells;
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
        } else {
            total_norm += number_outputs(d, li);
        }
    }
    /* Bernoulli masks: (AF units of the layer) * T per layer, in layer order
     * (Reset__Parameter__Mask_Dropout, NN/Neural_Network.cpp:3948-3962); LSTM layers own no AF unit. */
    uint64_t total_mask = 0;
    for (uint32_t li = 0; li < d->n_layers; ++li) {
        myea_layer_desc *l = &d->layers[li];
        l->first_mask_index = total_mask;
        if (l->type_layer == MYEA_LAYER_FULLY_CONNECTED) total_mask += (uint64_t)l->n_units * d->number_recurrent_depth;
    }
    d->total_weights = total_weights;
    d->total_bias = total_bias;
    d->total_normalized_units = any_norm ? total_norm : 0;
    d->total_parameters = total_weights + total_bias + 2u * d->total_normalized_units;
    d->total_mask_units = total_mask;
    return MYEA_OK;
}
