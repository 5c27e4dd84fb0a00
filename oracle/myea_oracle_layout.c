/* myea_oracle_layout.c — the index table of a compiled network, restated for the checker from the reference's own
 * Compile sequence.  TEST INFRASTRUCTURE ONLY: nothing in the product links or loads this.
 *
 * The walk below keeps the reference's order of operations and its bookkeeping - running counters of neuron units,
 * activation units, cells and blocks per layer, then connections, then biases, then normalised units, then masks - so that
 * the offsets come out of the same additions the reference performs:
 *   Assign__Layers / Assign__Residual_Block / Assign__Residual_Layer      NN/Neural_Network__Compile.cpp:20-223
 *   Organize__Previous_Layers_Connected                                    NN/Neural_Network.cpp:20-57
 *   Assign__Post__Layers / __Residual_Block / __Residual_Layer             NN/Neural_Network__Compile.cpp:225-420
 *   Prepare__Connections__FC / __FC_Ind_RNN / __LSTM, Prepare__Bias__*      NN/Neural_Network__Prepare_Connections.cpp:20-252,
 *                                                                          called from NN/Neural_Network__Compile.cpp:556-665
 *   Prepare__Normalized__Layers / __Residual_Block / __Residual_Layer      NN/Neural_Network__Layer_Normalization.cpp:20-150
 *   Reset__Parameter__Mask_Dropout                                         NN/Neural_Network.cpp:3948-3962
 * (NN/ = Neural_Network_Library_Windows/Source_Files/Neural_Network/.)
 * It exports the four descriptor helpers of include/myea_hip.h under their own names, so a test can hand the same
 * description to this file and to the product's layout code and compare the two tables field by field. */
#include <float.h>
#include <math.h>
#include <string.h>

#include "myea_oracle.h"

/* what Assign__Layer and Assign__Post__Layer leave in a struct Layer, as far as offsets depend on it */
typedef struct {
    uint64_t outputs;      /* *ptr_number_outputs */
    uint64_t neurons;      /* ptr_last_neuron_unit - ptr_array_neuron_units */
    uint64_t af_units;     /* AF_unit or AF_Ind_recurrent_unit count (a layer owns one kind) */
    uint64_t blocks, cells;/* LSTM: both directions together */
    uint32_t previous;     /* previous_connected_layers[0] */
    int in_block, first_in_block;
} walked_layer;

static int pooling(uint32_t type) { return type == MYEA_LAYER_AVERAGE_POOLING || type == MYEA_LAYER_MAX_POOLING; }
static int neuron_layer(uint32_t type) { return type == MYEA_LAYER_FULLY_CONNECTED || type == MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT; }

/* Organize__Previous_Layers_Connected over all layers: `state` is the residual layer whose block is being walked, `count`
 * the layers seen since it */
static void organize_previous(const myea_net_desc *d, walked_layer *w)
{
    long state = -1;
    uint32_t count = 0;
    for (uint32_t i = 0; i < d->n_layers; ++i) {
        w[i].in_block = 0; w[i].first_in_block = 0;
        if (i == 0) { w[i].previous = 0; }
        else if (state >= 0 && count++ == d->layers[state].block_depth) {   /* first layer behind a block: the residual layer */
            w[i].previous = (uint32_t)state;
            count = 0;
            state = -1;
        } else {
            uint32_t p = i - 1;
            if (d->layers[p].type_layer == MYEA_LAYER_RESIDUAL) p = w[p].previous;   /* first member: the shortcut source */
            w[i].previous = p;
            if (state >= 0) { w[i].in_block = 1; w[i].first_in_block = (long)i == state + 1; }
        }
        if (d->layers[i].type_layer == MYEA_LAYER_RESIDUAL) { state = (long)i; count = 0; }
    }
}

static int pooled_width(const myea_layer_desc *l, uint64_t in, uint64_t *out)
{
    /* floor or ceil of (in + 2 padding - kernel) / stride + 1 for the average, of (in + 2 padding - dilation (kernel - 1) - 1) / stride + 1
     * for the maximum, evaluated in unsigned arithmetic before the division as the reference writes it */
    const uint64_t kernel = l->pooling_values[0], stride = l->pooling_values[1], padding = l->pooling_values[2], dilation = l->pooling_values[3];
    if (kernel == 0 || stride == 0) return 0;
    const uint64_t plus = in + 2 * padding, minus = l->type_layer == MYEA_LAYER_AVERAGE_POOLING ? kernel : dilation * (kernel - 1) + 1;
    if (plus < minus) return 0;
    const double q = (double)(plus - minus) / (double)stride + 1.0;
    const double v = l->pooling_values[4] == 0 ? floor(q) : ceil(q);
    if (v < 1.0 || v > 4294967295.0) return 0;
    *out = (uint64_t)v;
    return 1;
}

static int walk(const myea_net_desc *d, walked_layer *w)
{
    organize_previous(d, w);
    /* Assign__Layer: units of the layers that state their own width */
    for (uint32_t i = 0; i < d->n_layers; ++i) {
        const myea_layer_desc *l = &d->layers[i];
        w[i].outputs = w[i].neurons = w[i].af_units = w[i].blocks = w[i].cells = 0;
        if (neuron_layer(l->type_layer)) {
            w[i].outputs = w[i].neurons = l->n_units;
            if (!w[i].in_block) w[i].af_units = l->n_units;          /* Assign__Residual_Layer gives a member no activation unit yet */
        } else if (l->type_layer == MYEA_LAYER_LSTM) {
            const uint64_t dirs = l->use_bidirectional ? 2 : 1;
            w[i].outputs = (uint64_t)l->n_units * l->n_cells_per_block;
            w[i].blocks = (uint64_t)l->n_units * dirs;
            w[i].cells = w[i].outputs * dirs;
        }
    }
    /* Assign__Post__Layer, in layer order: pooling widths, a residual layer's width, a member's activation units */
    for (uint32_t i = 1; i < d->n_layers; ++i) {
        const myea_layer_desc *l = &d->layers[i];
        if (pooling(l->type_layer)) {
            if (!pooled_width(l, w[w[i].previous].outputs, &w[i].outputs)) return MYEA_E_INVALID;
        } else if (l->type_layer == MYEA_LAYER_RESIDUAL) {
            /* the block's last layer must know its width first: members are walked from here (Assign__Post__Residual_Block) */
            const uint32_t last = i + l->block_depth;
            if (l->block_depth == 0 || last + 1 >= d->n_layers) return MYEA_E_INVALID;
            for (uint32_t m = i + 1; m <= last; ++m) {
                const myea_layer_desc *ml = &d->layers[m];
                if (pooling(ml->type_layer)) { if (!pooled_width(ml, w[w[m].previous].outputs, &w[m].outputs)) return MYEA_E_INVALID; }
                else if (neuron_layer(ml->type_layer)) { if (m != i + 1) w[m].af_units = w[w[m].previous].outputs; }   /* on the member's input side */
                else if (ml->type_layer != MYEA_LAYER_LSTM) return MYEA_E_UNSUPPORTED;   /* a block inside a block is not walked here */
            }
            const uint64_t a = w[w[i].previous].outputs, b = w[last].outputs;
            w[i].outputs = a > b ? a : b;
            i = last;
        }
    }
    return MYEA_OK;
}

void myea_hyper_default(myea_hyper *h)
{
    /* the public training fields as the constructor leaves them, Header_Files/Neural_Network/Data.hpp:2929-3060 */
    memset(h, 0, sizeof(*h));
    h->type_accuracy_function = MYEA_ACCURACY_DISTANCE;
    h->use_adam_bias_correction = 1;
    h->learning_rate = 0.01f; h->learning_rate_final = 0.1f; h->learning_momentum = 0.9f; h->learning_gamma = 1e-3f;
    h->adam_learning_rate = 0.001f; h->adam_beta1 = 0.9f; h->adam_beta2 = 0.999f; h->adam_epsilon = 1e-8f; h->adam_gamma = 0.1f;
    h->clip_gradient = 1.f;
    h->accuracy_variance = 0.49f; h->bit_fail_limit = 0.35f;
    h->normalization_momentum_average = 0.999f; h->normalization_epsilon = 1e-5f;
    h->batch_renormalization_r_correction_maximum = 1.f; h->batch_renormalization_d_correction_maximum = 0.f;
    h->use_normalized_weight_decay = 1; h->epoch_time_step = 1.f;
    h->rprop_increase_factor = 1.2f; h->rprop_decrease_factor = 0.5f; h->rprop_delta_min = 1e-6f; h->rprop_delta_max = 50.f; h->rprop_delta_zero = 0.1f;
    h->loss_rprop = FLT_MAX; h->previous_loss_rprop = FLT_MAX;
    h->warm_restarts_decay_learning_rate = 1.f; h->warm_restarts_maximum_learning_rate = 1.f; h->warm_restarts_minimum_learning_rate = 1e-7f;
    h->warm_restarts_T_i = 1.f; h->warm_restarts_multiplier = 2.f;
}

uint32_t myea_net_desc_previous_layer(const myea_net_desc *d, uint32_t li)
{
    walked_layer w[MYEA_MAX_LAYERS];
    if (!d || li == 0 || li >= d->n_layers || d->n_layers > MYEA_MAX_LAYERS) return 0;
    organize_previous(d, w);
    return w[li].previous;
}

uint64_t myea_net_desc_number_outputs(const myea_net_desc *d, uint32_t li)
{
    walked_layer w[MYEA_MAX_LAYERS];
    if (!d || li >= d->n_layers || d->n_layers > MYEA_MAX_LAYERS) return 0;
    /* widths of pooling layers are part of the description once it has been laid out; before that they are computed */
    if (walk(d, w) != MYEA_OK) return 0;
    return w[li].outputs;
}

int myea_net_desc_layout(myea_net_desc *d)
{
    walked_layer w[MYEA_MAX_LAYERS];
    if (!d || d->n_layers < 2 || d->n_layers > MYEA_MAX_LAYERS || d->number_recurrent_depth == 0 || d->batch_size == 0) return MYEA_E_INVALID;
    for (uint32_t i = 0; i < d->n_layers; ++i) {
        const myea_layer_desc *l = &d->layers[i];
        const int known = neuron_layer(l->type_layer) || l->type_layer == MYEA_LAYER_LSTM || l->type_layer == MYEA_LAYER_RESIDUAL || pooling(l->type_layer);
        if (!known) return MYEA_E_UNSUPPORTED;
        if ((neuron_layer(l->type_layer) || l->type_layer == MYEA_LAYER_LSTM) && l->n_units == 0) return MYEA_E_INVALID;
        if (l->type_layer == MYEA_LAYER_LSTM && l->n_cells_per_block == 0) return MYEA_E_INVALID;
        if ((i == 0 || i + 1 == d->n_layers) && l->type_layer != MYEA_LAYER_FULLY_CONNECTED) return MYEA_E_INVALID;
        if (l->k_sparsity != 0) {
            /* Set__K_Sparsity / Set__Alpha_Sparsity, NN/Neural_Network__K_Sparse.cpp:38-190 */
            const float scaled = (float)l->k_sparsity * l->alpha_sparsity;
            if (i == 0 || i + 1 == d->n_layers || l->type_layer != MYEA_LAYER_FULLY_CONNECTED) return MYEA_E_UNSUPPORTED;
            if (l->k_sparsity > l->n_units || !(l->alpha_sparsity >= 0.f) || !(scaled >= 1.f) || (uint64_t)scaled > l->n_units) return MYEA_E_INVALID;
        }
    }
    {
        const int rc = walk(d, w);
        if (rc != MYEA_OK) return rc;
    }
    for (uint32_t i = 1; i < d->n_layers; ++i)
        if (pooling(d->layers[i].type_layer)) d->layers[i].n_units = (uint32_t)w[i].outputs;

    /* connections, layer by layer behind the input layer (Compile.cpp:556-620): pooling and residual layers own none */
    uint64_t total_weights = 0;
    for (uint32_t i = 1; i < d->n_layers; ++i) {
        myea_layer_desc *l = &d->layers[i];
        const uint64_t fan_in = w[w[i].previous].outputs;
        uint64_t allocated = 0;
        l->first_connection_index = total_weights;
        if (neuron_layer(l->type_layer)) {
            allocated = w[i].neurons * fan_in;                                                        /* Prepare__Connections__FC */
            if (l->type_layer == MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT) allocated += w[i].af_units;   /* one self connection per recurrent activation unit */
        } else if (l->type_layer == MYEA_LAYER_LSTM) {
            const uint64_t per_layer_cells = w[i].cells >> (l->use_bidirectional ? 1 : 0), per_layer_blocks = w[i].blocks >> (l->use_bidirectional ? 1 : 0);
            const uint64_t cells_per_block = per_layer_cells / per_layer_blocks;
            for (uint64_t b = 0; b < w[i].blocks; ++b) {
                allocated += cells_per_block * (fan_in + per_layer_cells);   /* every cell: block input from below, then recurrent */
                allocated += 3 * fan_in;                                       /* input, forget, output gate from below */
                allocated += 3 * per_layer_cells;                              /* ... recurrent */
                allocated += 3 * cells_per_block;                              /* peepholes */
            }
        }
        total_weights += allocated;
        l->last_connection_index = total_weights;
    }
    /* biases (Compile.cpp:622-660).  Prepare__Bias__LSTM assigns first_bias_connection_index twice: the value that stays is
     * the start of the layer's slice plus its cell count. */
    uint64_t total_bias = 0;
    for (uint32_t i = 1; i < d->n_layers; ++i) {
        myea_layer_desc *l = &d->layers[i];
        l->first_bias_connection_index = total_weights + total_bias;
        if (neuron_layer(l->type_layer)) total_bias += w[i].outputs;
        else if (l->type_layer == MYEA_LAYER_LSTM) {
            /* two directions: this library's own contract (the reference overlays the directions): the slice starts at its
             * start, direction 1's vectors follow direction 0's */
            if (!l->use_bidirectional) l->first_bias_connection_index += w[i].cells;
            total_bias += w[i].cells + 3 * w[i].blocks;
        }
    }
    d->layers[0].first_connection_index = d->layers[0].last_connection_index = d->layers[0].first_bias_connection_index = 0;
    /* normalised units, every layer in order, the input layer included (Prepare__Normalized__Layers) */
    uint64_t total_norm = 0;
    int any_norm = 0;
    for (uint32_t i = 0; i < d->n_layers; ++i) {
        myea_layer_desc *l = &d->layers[i];
        l->first_normalized_unit_index = total_norm;
        if (l->type_normalization != MYEA_NORMALIZATION_NONE) any_norm = 1;
        if (neuron_layer(l->type_layer)) total_norm += w[i].in_block ? w[w[i].previous].outputs : w[i].outputs;
        else if (l->type_layer == MYEA_LAYER_LSTM) total_norm += 3 * w[i].cells + 6 * w[i].blocks;
        else if (l->type_layer == MYEA_LAYER_RESIDUAL) total_norm += w[i + l->block_depth].outputs;
    }
    /* Bernoulli masks: (activation units of the layer) x T, in layer order */
    uint64_t total_mask = 0;
    for (uint32_t i = 0; i < d->n_layers; ++i) {
        d->layers[i].first_mask_index = total_mask;
        total_mask += w[i].af_units * d->number_recurrent_depth;
    }
    d->total_weights = total_weights;
    d->total_bias = total_bias;
    d->total_normalized_units = any_norm ? total_norm : 0;   /* the scale / shift region exists once a layer is normalised, NN/Neural_Network__Allocate.cpp:2378-2406 */
    d->total_parameters = total_weights + total_bias + 2 * d->total_normalized_units;
    d->total_mask_units = total_mask;
    return MYEA_OK;
}
