/* myea_oracle.c — CPU restatement of the reference's training step.  TEST INFRASTRUCTURE ONLY:
 * only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this.
 *
 * Each function follows the reference file:line named above it.  Abbreviations:
 *   NN/  = Neural_Network_Library_Windows/Source_Files/Neural_Network/
 *   NNH/ = Neural_Network_Library_Windows/Header_Files/Neural_Network/
 *
 * The reference itself cannot be built in this image (every translation unit includes
 * Header_Files/stdafx.hpp -> <Eigen/QR>, Configuration.hpp -> <boost/assert.hpp>,
 * Dataset_Manager.hpp -> <systemd/sd-bus.h>; none of the three is installed or vendored), and it
 * ships no tests, golden vectors or fixtures.  This restatement is therefore pinned by what the
 * mathematics fixes — see tests/test_oracle_*.py: automatic differentiation of an independent
 * float64 forward model, closed forms, brute force on tiny shapes and invariants.
 * Parts of the behaviour that are reference quirks rather than mathematics (listed at each
 * function) are pinned only by reading: "parity unpinned" for
 *   - the LSTM bias index overrun (Prepare__Bias__LSTM),
 *   - the RNN head `pre` pointer quirk (RNN__Compute__Error),
 *   - the Nesterov update sign, ELU' / SELU' as written, the backward pass having no dropout, zoneout, k-sparse or
 *     noise-dropout operator (each restated as written, with a test that shows where it leaves the textbook form),
 *   - which of several EQUAL values stays at a k-sparse filter's cut (std::sort's order in the reference; the lower
 *     index here),
 *   - the random draws of Gaussian / Uout dropout and ShakeDrop: an INPUT of this restatement (the reference draws them
 *     from its host generators inside the pass).
 *
 * Summation order is the serial order of the reference's __Loop variants; the __OpenMP variants
 * differ only in the order of the per-thread partial sums.
 */
#include "myea_oracle.h"

#include <float.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* LSTM-with-peephole layer state, one direction.  Cell tensors are [T][Bmax][C], block tensors [T][Bmax][K]
 * (NNH/Data.hpp:2985-3016: ptr_array_cells_* / ptr_array_blocks_*). */
typedef struct olstm {
    size_t K, cpb, C, In;   /* blocks, cells per block, cells, fan-in (per direction) */
    size_t per_block;       /* parameters of one block */
    size_t base, bias;      /* flat index of the direction's first block and of its bias vectors z | i | f | o */
    int reverse;            /* the direction walks time from T-1 down to 0 */
    const uint8_t *zone_state, *zone_output;   /* zoneout masks of the direction: [T][zone_stride], this direction's cells first at 0 */
    size_t zone_stride;
    float *h, *dh;          /* cell outputs and their delta [T][Bmax][C]: the layer's own buffers for a one-direction layer */
    float *sum_in_z, *sum_rec_z, *sum_z, *z, *c, *ca;          /* cells */
    float *sum_in_i, *sum_in_f, *sum_in_o, *sum_rec_i, *sum_rec_f, *sum_rec_o, *sum_i, *sum_f, *sum_o, *gi, *gf, *go; /* blocks */
    float *dz, *dc, *di, *df, *dgo;                              /* deltas */
    /* normalised layer (NN/Neural_Network__Allocate.cpp:2710-2790, one cell per block): nine groups of normalised units,
     * 0 block input from below, 1 block input recurrent, 2 cell state, 3 / 4 input gate, 5 / 6 forget gate, 7 / 8 output gate
     * (from below / recurrent), each with its own statistics per time step; and the deltas of the eight sums after the
     * backward pass through their normalisation */
    int norm;
    struct obn {
        size_t H, param;   /* width; flat index of the group's first scale (the shift sits total_normalized_units further) */
        float *means, *variances, *means_averages, *variances_averages, *r_corrections, *d_corrections;   /* [T][H] */
        float *derivatives_means, *derivatives_variances;
        float *hats, *normalizes;   /* [T][Bmax][H] */
    } nrm[9];
    float *dz_in, *dz_rec, *di_in, *di_rec, *df_in, *df_rec, *do_in, *do_rec;
} olstm;
typedef struct obn obn;

typedef struct olayer {
    size_t H;            /* *ptr_number_outputs */
    size_t norm_units;   /* number of Normalized_unit owned by the layer */
    /* topology (Organize__Previous_Layers_Connected / Organize__Layer__Group, NN/Neural_Network.cpp:20-125) */
    size_t prev;         /* previous_connected_layers[0] */
    int group;           /* 0 outside a residual block, 1 first layer of a block, 2 other layers of a block */
    size_t In;           /* *previous_connected_layers[0]->ptr_number_outputs */
    size_t AH, NH;       /* width of the AF-unit tensors (values, af_errors) and of the normalised-unit tensors:
                            H outside a block; inside a block they sit on the input side and are In wide; a residual
                            layer has basic units (H wide, kept in values / af_errors) and NH = the block's last width */
    size_t pad;          /* residual layer: pooling_values[2], the zero-padding offset of the narrower operand */
    /* [T][Bmax][H] (summations, neuron_errors), [T][Bmax][AH] (values, af_errors), [T][Bmax][NH] (hats, normalizes, norm_errors) */
    float *summations, *values, *hats, *normalizes;
    float *neuron_errors, *af_errors, *norm_errors;
    /* [T][NH] */
    float *means, *variances, *means_averages, *variances_averages, *r_corrections, *d_corrections;
    float *derivatives_means, *derivatives_variances;
    /* per-unit activation types / steepnesses (AF_unit arrays), NULL = the layer-wide value; AH entries */
    uint32_t *unit_af; float *unit_steep;
    /* LSTM: one olstm per direction */
    struct olstm *lstm;
    /* max pooling: Basic_indice_unit::ptr_array_indices, the (padded) position each output took its value from [T][Bmax][H] */
    uint32_t *pool_index;
    /* independently recurrent layer: AF_Ind_recurrent_unit::ptr_array_pre_AFs and ::ptr_array_dAFs [T][Bmax][H]
     * (its ptr_array_AFs are `values`, its ptr_array_errors `af_errors`) */
    float *pre_afs, *dafs;
    /* Gaussian / Uout dropout: the draws of the forward pass [T][Bmax][H], supplied by the test (the reference draws them from
     * its host generators inside the pass); all-neutral after create */
    float *noise;
} olayer;

struct myea_oracle_net {
    myea_net_desc d;
    myea_hyper h;
    uint32_t state;
    int threads;
    float *parameters, *gradient, *opt[MYEA_STATE_KINDS];
    uint8_t *masks;
    uint8_t *zoneout; size_t zoneout_count;   /* ptr_array_cell_units_mask_dropout_zoneout: state half, then output half */
    olayer L[MYEA_MAX_LAYERS];
    myea_loss_state loss;
};

/* ------------------------------------------------------------------------------------------- */
/* activation functions: NNH/Activation_Functions.hpp:17-184 (AF_FIRE; forward ignores steepness) */

static float af_linear_seg(float v1, float r1, float v2, float r2, float s) { return (((r2 - r1) * (s - v1)) / (v2 - v1)) + r1; }

static float af_stepwise(float v1, float v2, float v3, float v4, float v5, float v6,
                         float r1, float r2, float r3, float r4, float r5, float r6,
                         float mn, float mx, float s)
{
    return s < v5 ? (s < v3 ? (s < v2 ? (s < v1 ? mn : af_linear_seg(v1, r1, v2, r2, s)) : af_linear_seg(v2, r2, v3, r3, s))
                            : (s < v4 ? af_linear_seg(v3, r3, v4, r4, s) : af_linear_seg(v4, r4, v5, r5, s)))
                  : (s < v6 ? af_linear_seg(v5, r5, v6, r6, s) : mx);
}

#define SELU_ALPHA 1.6732632423543772848170429916717f
#define SELU_SCALE 1.0507009873554804934193349852946f

float myea_oracle_activation(uint32_t type, float s)
{
    switch (type) {
    case MYEA_AF_LINEAR: return s;
    case MYEA_AF_LINEAR_PIECE: return s < 0.f ? 0.f : (s > 1.f ? 1.f : s);
    case MYEA_AF_LINEAR_PIECE_SYMMETRIC: return s < -1.f ? -1.f : (s > 1.f ? 1.f : s);
    case MYEA_AF_SIGMOID: return 1.f / (1.f + expf(-s));                      /* AF_SIGMOID_real */
    case MYEA_AF_TANH: return 2.f / (1.f + expf(-2.f * s)) - 1.f;             /* AF_TANH_real (not tanhf) */
    case MYEA_AF_SIGMOID_STEPWISE:
        return af_stepwise(-2.64665246009826660156f, -1.47221946716308593750f, -5.49306154251098632812e-01f,
                           5.49306154251098632812e-01f, 1.47221934795379638672f, 2.64665293693542480469f,
                           4.99999988824129104614e-03f, 5.00000007450580596924e-02f, 2.5e-01f, 7.5e-01f,
                           9.49999988079071044922e-01f, 9.95000004768371582031e-01f, 0.f, 1.f, s);
    case MYEA_AF_TANH_STEPWISE:
        return af_stepwise(-2.64665293693542480469f, -1.47221934795379638672f, -5.49306154251098632812e-01f,
                           5.49306154251098632812e-01f, 1.47221934795379638672f, 2.64665293693542480469f,
                           -9.90000009536743164062e-01f, -8.99999976158142089844e-01f, -5.0e-01f, 5.0e-01f,
                           8.99999976158142089844e-01f, 9.90000009536743164062e-01f, -1.f, 1.f, s);
    case MYEA_AF_THRESHOLD: return s < 0.f ? 0.f : 1.f;
    case MYEA_AF_THRESHOLD_SYMMETRIC: return s < 0.f ? -1.f : 1.f;
    case MYEA_AF_GAUSSIAN: return expf(-s * s);
    case MYEA_AF_GAUSSIAN_SYMMETRIC: return expf(-s * s) * 2.f - 1.f;
    case MYEA_AF_GAUSSIAN_STEPWISE: return 0.f;
    case MYEA_AF_ELLIOT: return (s / 2.f) / (1.f + fabsf(s)) + 0.5f;
    case MYEA_AF_ELLIOT_SYMMETRIC: return s / (1.f + fabsf(s));
    case MYEA_AF_SINE: return sinf(s) / 2.f + 0.5f;
    case MYEA_AF_SINE_SYMMETRIC: return sinf(s);
    case MYEA_AF_COSINE: return cosf(s) / 2.f + 0.5f;
    case MYEA_AF_COSINE_SYMMETRIC: return cosf(s);
    case MYEA_AF_ISRU: return s * (1.f / sqrtf(1.f + 1.f * s * s));
    case MYEA_AF_ISRLU: return s < 0.f ? s * (1.f / sqrtf(1.f + 1.f * s * s)) : s;
    case MYEA_AF_ELU: return s < 0.f ? 1.f * (expf(s) - 1.f) : s;
    case MYEA_AF_SELU: return SELU_SCALE * (s <= 0.f ? SELU_ALPHA * expf(s) - SELU_ALPHA : s);
    case MYEA_AF_RELU: return s < 0.f ? 0.f : s;
    case MYEA_AF_LEAKY_RELU: return s < 0.f ? 0.01f * s : s;
    case MYEA_AF_PARAMETRIC_RELU: return s < 0.f ? 0.01f * s : s;
    case MYEA_AF_SOFTMAX: return expf(s);
    default: return s; /* AF_FIRE default: leaves the value untouched */
    }
}

/* Activation_Function_Derive: NN/Neural_Network.cpp:3157-3201 + the *_derive macros. */
float myea_oracle_activation_derive(uint32_t type, float q, float st, float v)
{
    switch (type) {
    case MYEA_AF_COSINE: return st * -sinf(st * q) / 2.f;
    case MYEA_AF_COSINE_SYMMETRIC: return st * -sinf(st * q);
    case MYEA_AF_ELU: return q < 0.f ? st * 1.f * v : st;
    case MYEA_AF_ELLIOT: return st * 1.f / (2.f * (1.f + fabsf(q)) * (1.f + fabsf(q)));
    case MYEA_AF_ELLIOT_SYMMETRIC: return st * 1.f / ((1.f + fabsf(q)) * (1.f + fabsf(q)));
    case MYEA_AF_GAUSSIAN: return -2.f * q * v * st * st;
    case MYEA_AF_GAUSSIAN_SYMMETRIC: return -2.f * q * (v + 1.f) * st * st;
    /* static_cast<T_>(pow(value / summation, 3u)): the float quotient is cubed in double and rounded once (Activation_Functions.hpp:86, 90) */
    case MYEA_AF_ISRU: { float r = v / q; return st * (float)pow((double)r, 3.0); }
    case MYEA_AF_ISRLU: { float r = v / q; return q < 0.f ? st * (float)pow((double)r, 3.0) : st; }
    case MYEA_AF_LINEAR:
    case MYEA_AF_LINEAR_PIECE:
    case MYEA_AF_LINEAR_PIECE_SYMMETRIC: return st;
    case MYEA_AF_LEAKY_RELU: return q < 0.f ? st * 0.01f : st;
    case MYEA_AF_PARAMETRIC_RELU: return q < 0.f ? st * 0.01f : st;
    case MYEA_AF_RELU: return q < 0.f ? 0.f : st;          /* 1 at q == 0 */
    case MYEA_AF_SELU: return SELU_SCALE * (q <= 0.f ? st * (v + SELU_ALPHA) : st);
    case MYEA_AF_SIGMOID:
    case MYEA_AF_SIGMOID_STEPWISE: return st * v * (1.f - v);
    case MYEA_AF_SINE: return st * cosf(st * q) / 2.f;
    case MYEA_AF_SINE_SYMMETRIC: return st * cosf(st * q);
    case MYEA_AF_TANH:
    case MYEA_AF_TANH_STEPWISE: return st * (1.f - v * v);
    case MYEA_AF_SOFTMAX: return st;                       /* cross-entropy shortcut */
    default: return v;
    }
}

/* ------------------------------------------------------------------------------------------- */
/* helpers */

static int layer_uses_norm(const myea_layer_desc *l) { return l->type_normalization != MYEA_NORMALIZATION_NONE; }
static int is_ind_rnn(const myea_layer_desc *l) { return l->type_layer == MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT; }
/* layers made of neuron units and activation units */
static int is_dense(const myea_layer_desc *l) { return l->type_layer == MYEA_LAYER_FULLY_CONNECTED || is_ind_rnn(l); }
static int layer_uses_bias(const myea_layer_desc *l) { return !layer_uses_norm(l); } /* NNH/Data.hpp:736 */

static float *zalloc(size_t n) { return (float *)calloc(n ? n : 1, sizeof(float)); }

/* Layer::ptr_array_outputs, NN/Neural_Network__Ordered.cpp:78-389 (non-residual group). */
static float *layer_outputs(myea_oracle_net *n, size_t li)
{
    const myea_layer_desc *l = &n->d.layers[li];
    olayer *o = &n->L[li];
    if (li == 0) return o->values;
    if (is_dense(l)) {
        if (o->group) return o->summations; /* residual group: NN/Neural_Network__Ordered.cpp:96-141 */
        if (layer_uses_norm(l) && !l->use_layer_normalization_before_activation) return o->normalizes;
        return o->values;
    }
    return o->values; /* LSTM: cell outputs live in values; residual layer: basic units' values (:360-366) */
}

/* Layer::ptr_array_derivative_outputs */
static float *layer_derivative_outputs(myea_oracle_net *n, size_t li)
{
    const myea_layer_desc *l = &n->d.layers[li];
    olayer *o = &n->L[li];
    if (is_dense(l)) {
        if (o->group) return o->neuron_errors;
        if (layer_uses_norm(l) && !l->use_layer_normalization_before_activation) return o->norm_errors;
        return o->af_errors;
    }
    return o->af_errors; /* LSTM: ptr_delta_cell_output; residual layer: basic units' errors */
}

static float *scale_ptr(myea_oracle_net *n, float *base, size_t li)
{
    return base + n->d.total_weights + n->d.total_bias + n->d.layers[li].first_normalized_unit_index;
}
static float *shift_ptr(myea_oracle_net *n, float *base, size_t li)
{
    return scale_ptr(n, base, li) + n->d.total_normalized_units;
}

/* ------------------------------------------------------------------------------------------- */
/* life cycle */

static int is_pooling(const myea_layer_desc *l) { return l->type_layer == MYEA_LAYER_AVERAGE_POOLING || l->type_layer == MYEA_LAYER_MAX_POOLING; }

static size_t layer_width(const myea_layer_desc *l)
{
    if (l->type_layer == MYEA_LAYER_LSTM) return (size_t)l->n_units * l->n_cells_per_block;
    return l->n_units;
}

int myea_oracle_create(const myea_net_desc *desc, myea_oracle_net **out)
{
    if (!desc || !out || desc->n_layers < 2 || desc->n_layers > MYEA_MAX_LAYERS) return MYEA_E_INVALID;
    myea_oracle_net *n = (myea_oracle_net *)calloc(1, sizeof(*n));
    if (!n) return MYEA_E_NOMEM;
    n->d = *desc;
    /* a pooling layer may carry a normalisation type (the reference's setter takes any hidden layer, Neural_Network__Layer_
     * Normalization.cpp:217-288; its example program sets one on every hidden layer): the layer owns no normalised unit and
     * its passes never look at the field, so this copy of the description drops it */
    for (size_t li = 0; li < n->d.n_layers; ++li)
        if (n->d.layers[li].type_layer == MYEA_LAYER_AVERAGE_POOLING || n->d.layers[li].type_layer == MYEA_LAYER_MAX_POOLING) n->d.layers[li].type_normalization = MYEA_NORMALIZATION_NONE;
    desc = &n->d;
    myea_hyper_default(&n->h);
    n->threads = 1;
    size_t P = desc->total_parameters, T = desc->number_recurrent_depth, B = desc->batch_size;
    n->parameters = zalloc(P);
    n->gradient = zalloc(P);
    for (int k = 0; k < MYEA_STATE_KINDS; ++k) n->opt[k] = zalloc(P);
    for (size_t i = 0; i < P; ++i) n->opt[MYEA_STATE_PREVIOUS_STEPS][i] = n->h.rprop_delta_zero;   /* the iRPROP steps start at delta zero */
    n->masks = (uint8_t *)malloc(desc->total_mask_units ? desc->total_mask_units : 1);
    memset(n->masks, 1, desc->total_mask_units ? desc->total_mask_units : 1); /* NN/Neural_Network__Allocate.cpp:386-410: all true */
    /* scales start at 1, shifts at 0 (NN/Neural_Network__Allocate.cpp:2395-2401 and the scale fill) */
    for (size_t i = 0; i < desc->total_normalized_units; ++i) n->parameters[desc->total_weights + desc->total_bias + i] = 1.f;
    /* connections, walked with the same running state as Order__Layers__Connection (NN/Neural_Network__Ordered.cpp:20-68):
     * `block` is the residual layer whose members are being visited, `seen` how many of them have been */
    {
        size_t block = 0, seen = 0;
        for (size_t li = 0; li < desc->n_layers; ++li) {
            const myea_layer_desc *l = &desc->layers[li];
            olayer *o = &n->L[li];
            o->group = 0;
            if (li == 0) { o->prev = 0; o->H = l->n_units; if (l->type_layer == MYEA_LAYER_RESIDUAL) { free(n); return MYEA_E_INVALID; } continue; }
            if (block != 0 && seen == desc->layers[block].block_depth) { o->prev = block; block = 0; seen = 0; } /* first layer after the block */
            else {
                o->prev = li - 1;
                if (desc->layers[li - 1].type_layer == MYEA_LAYER_RESIDUAL) o->prev = n->L[li - 1].prev;
                if (block != 0) { o->group = seen == 0 ? 1 : 2; ++seen; }
            }
            if (l->type_layer == MYEA_LAYER_RESIDUAL) {
                if (block != 0 || l->block_depth == 0 || li + l->block_depth + 1 >= desc->n_layers || (l->type_dropout != MYEA_DROPOUT_NONE && l->type_dropout != MYEA_DROPOUT_SHAKEDROP)) { free(n); return MYEA_E_UNSUPPORTED; }
                block = li; seen = 0;
            }
        }
        /* widths: a residual layer is as wide as the wider of its shortcut source and its block's last layer
         * (Assign__Post__Layer, NN/Neural_Network__Compile.cpp:272-281); its members' widths are known up front */
        for (size_t li = 0; li < desc->n_layers; ++li) {
            const myea_layer_desc *l = &desc->layers[li];
            olayer *o = &n->L[li];
            if (l->type_layer == MYEA_LAYER_RESIDUAL) {
                size_t a = n->L[o->prev].H, b = layer_width(&desc->layers[li + l->block_depth]);
                o->H = a > b ? a : b;
                o->pad = ((a > b ? a - b : b - a) + 1) / 2;
                o->NH = b;
            } else o->H = layer_width(l);
            o->In = li ? n->L[o->prev].H : 0;
            if (is_pooling(l) || l->type_layer == MYEA_LAYER_LSTM) { o->AH = o->H; o->NH = o->H; }   /* basic units / cells: as wide as the layer, inside a block too */
            else if (l->type_layer != MYEA_LAYER_RESIDUAL) { o->AH = o->group ? (o->group == 1 ? 0 : o->In) : o->H; o->NH = o->group ? o->In : o->H; }
            else o->AH = o->H;
        }
    }
    size_t total_cells = 0, zone_at = 0;
    for (size_t li = 0; li < desc->n_layers; ++li)
        if (desc->layers[li].type_layer == MYEA_LAYER_LSTM) total_cells += (size_t)desc->layers[li].n_units * desc->layers[li].n_cells_per_block * (desc->layers[li].use_bidirectional ? 2 : 1);
    n->zoneout_count = 2 * T * total_cells;
    n->zoneout = (uint8_t *)malloc(n->zoneout_count ? n->zoneout_count : 1);
    memset(n->zoneout, 1, n->zoneout_count ? n->zoneout_count : 1);
    for (size_t li = 0; li < desc->n_layers; ++li) {
        const myea_layer_desc *l = &desc->layers[li];
        olayer *o = &n->L[li];
        /* members of a residual block: fully-connected, independently recurrent, LSTM and pooling layers (the recurrent member
         * switch, NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:711-771).  An independently recurrent member that is not
         * the block's first carries its recurrence on its input side, fan-in wide; the reference's backward pass walks those
         * units with the member's OUTPUT width (NN/Neural_Network__Backward_Pass__OpenMP.cpp:867-877 hands tmp_output_size to
         * Backward_Pass__FC__DF_Ind_RNN), which addresses them correctly only when the two widths are equal: other shapes have no
         * behaviour to follow */
        if (o->group == 2 && is_ind_rnn(l) && o->In != o->H) { free(n); return MYEA_E_UNSUPPORTED; }
        if (l->type_layer == MYEA_LAYER_LSTM && l->type_dropout != MYEA_DROPOUT_NONE && l->type_dropout != MYEA_DROPOUT_ZONEOUT) { free(n); return MYEA_E_UNSUPPORTED; }
        /* with more cells per block the reference's indices [3] .. [8] into the layer's normalised units (NN/Neural_Network.cpp:4498-4613)
         * land on the second cell's units instead of the block's (the units are laid out per block: 3 per cell, then 6,
         * NN/Neural_Network__Ordered.cpp:937-966): no behaviour to follow */
        if (l->type_layer == MYEA_LAYER_LSTM && layer_uses_norm(l) && l->n_cells_per_block != 1) { free(n); return MYEA_E_UNSUPPORTED; }
        if (l->type_layer != MYEA_LAYER_LSTM && l->type_dropout == MYEA_DROPOUT_ZONEOUT) { free(n); return MYEA_E_UNSUPPORTED; }
        if (is_ind_rnn(l) && l->type_activation_function == MYEA_AF_SOFTMAX) { free(n); return MYEA_E_UNSUPPORTED; }
        size_t sz = T * B * o->H;
        o->values = zalloc(T * B * o->AH);
        if (li == 0) continue;
        if (l->type_layer == MYEA_LAYER_LSTM) {
            /* the bias vectors are read at first_bias_connection_index + [0, C + 3K): with the index as the reference
             * leaves it they run C entries past the layer's own slice; past the end of the bias region the reference
             * reads and writes outside its parameter array, which nothing here reproduces */
            if (l->first_bias_connection_index + (l->use_bidirectional ? 2u : 1u) * ((size_t)l->n_units * l->n_cells_per_block + 3u * l->n_units) > desc->total_weights + desc->total_bias) { free(n); return MYEA_E_INVALID; }
            size_t dirs = l->use_bidirectional ? 2 : 1;
            olstm *qq = (olstm *)calloc(2, sizeof(olstm));
            o->af_errors = zalloc(sz);  /* ptr_delta_cell_output */
            for (size_t dir = 0; dir < dirs; ++dir) {
                olstm *q = &qq[dir];
                q->K = l->n_units; q->cpb = l->n_cells_per_block; q->C = q->K * q->cpb; q->In = o->In;
                q->per_block = q->cpb * (q->In + q->C) + 3 * q->In + 3 * q->C + 3 * q->cpb;
                q->base = l->first_connection_index + dir * q->K * q->per_block;
                q->bias = l->first_bias_connection_index + dir * (q->C + 3 * q->K);
                q->reverse = (int)dir;
                q->zone_stride = q->C * dirs;
                q->zone_state = n->zoneout + zone_at + dir * q->C;
                q->zone_output = q->zone_state + T * total_cells;
                size_t sc = T * B * q->C, sk = T * B * q->K;
                float **cells[] = {&q->sum_in_z, &q->sum_rec_z, &q->sum_z, &q->z, &q->c, &q->ca, &q->dz, &q->dc};
                float **blocks[] = {&q->sum_in_i, &q->sum_in_f, &q->sum_in_o, &q->sum_rec_i, &q->sum_rec_f, &q->sum_rec_o, &q->sum_i, &q->sum_f, &q->sum_o,
                                    &q->gi, &q->gf, &q->go, &q->di, &q->df, &q->dgo};
                for (size_t a = 0; a < sizeof(cells) / sizeof(cells[0]); ++a) *cells[a] = zalloc(sc);
                for (size_t a = 0; a < sizeof(blocks) / sizeof(blocks[0]); ++a) *blocks[a] = zalloc(sk);
                if (dirs == 2) { q->h = zalloc(sc); q->dh = zalloc(sc); }
                else { q->h = o->values; q->dh = o->af_errors; }
                q->norm = layer_uses_norm(l);
                if (q->norm) {
                    /* scales of the layer: per direction [3 groups of C | 6 groups of K] in group order (Allocate: the scale
                     * iterator advances group by group, :2718-2776) */
                    size_t at = desc->total_weights + desc->total_bias + l->first_normalized_unit_index + dir * (3 * q->C + 6 * q->K);
                    for (int g = 0; g < 9; ++g) {
                        obn *bn = &q->nrm[g];
                        bn->H = g < 3 ? q->C : q->K;
                        bn->param = at; at += bn->H;
                        float **small[] = {&bn->means, &bn->variances, &bn->means_averages, &bn->variances_averages, &bn->r_corrections, &bn->d_corrections,
                                           &bn->derivatives_means, &bn->derivatives_variances};
                        for (size_t a = 0; a < sizeof(small) / sizeof(small[0]); ++a) *small[a] = zalloc(T * bn->H);
                        for (size_t a = 0; a < T * bn->H; ++a) bn->variances_averages[a] = 1.f;   /* NN/Neural_Network__Allocate.cpp:2612-2615 */
                        bn->hats = zalloc(T * B * bn->H); bn->normalizes = zalloc(T * B * bn->H);
                    }
                    float **dc_[] = {&q->dz_in, &q->dz_rec}, **dk_[] = {&q->di_in, &q->di_rec, &q->df_in, &q->df_rec, &q->do_in, &q->do_rec};
                    for (size_t a = 0; a < 2; ++a) *dc_[a] = zalloc(sc);
                    for (size_t a = 0; a < 6; ++a) *dk_[a] = zalloc(sk);
                }
            }
            o->lstm = qq;
            zone_at += T * qq[0].zone_stride;
            continue;
        }
        o->af_errors = zalloc(T * B * o->AH);
        if (is_pooling(l)) {   /* basic (indice) units: values and errors only */
            if (l->type_layer == MYEA_LAYER_MAX_POOLING) o->pool_index = (uint32_t *)calloc(sz ? sz : 1, sizeof(uint32_t));
            continue;
        }
        if (l->type_layer != MYEA_LAYER_RESIDUAL) {
            o->summations = zalloc(sz);
            o->neuron_errors = zalloc(sz);
        }
        if (is_ind_rnn(l)) { o->pre_afs = zalloc(o->group ? T * B * o->AH : sz); o->dafs = zalloc(o->group ? T * B * o->AH : sz); }
        if (l->type_layer == MYEA_LAYER_RESIDUAL && l->type_dropout == MYEA_DROPOUT_SHAKEDROP) o->noise = zalloc(T * (B + 2 * B * o->NH));   /* all masks false */
        if (l->type_layer != MYEA_LAYER_RESIDUAL && l->type_dropout == MYEA_DROPOUT_SHAKEDROP) { free(n); return MYEA_E_UNSUPPORTED; }
        if (l->type_dropout == MYEA_DROPOUT_GAUSSIAN || l->type_dropout == MYEA_DROPOUT_UOUT) {
            /* one draw per activation unit: the layer's own width, or a block member's fan-in (none for a block's first member) */
            if (l->type_layer != MYEA_LAYER_FULLY_CONNECTED || o->group == 1) { free(n); return MYEA_E_UNSUPPORTED; }
            size_t sa = T * B * o->AH;
            o->noise = zalloc(sa);
            if (l->type_dropout == MYEA_DROPOUT_GAUSSIAN) for (size_t i = 0; i < sa; ++i) o->noise[i] = 1.f;
        }
        if (layer_uses_norm(l)) {
            size_t sn = T * B * o->NH, tn = T * o->NH;
            o->hats = zalloc(sn);
            o->normalizes = zalloc(sn);
            o->norm_errors = zalloc(sn);
            o->means = zalloc(tn);
            o->variances = zalloc(tn);
            o->means_averages = zalloc(tn);
            o->variances_averages = zalloc(tn);
            for (size_t i = 0; i < tn; ++i) o->variances_averages[i] = 1.f; /* NN/Neural_Network__Allocate.cpp:2612-2615 */
            o->r_corrections = zalloc(tn);
            o->d_corrections = zalloc(tn);
            o->derivatives_means = zalloc(tn);
            o->derivatives_variances = zalloc(tn);
        }
    }
    *out = n;
    return MYEA_OK;
}

int myea_oracle_destroy(myea_oracle_net *n)
{
    if (!n) return MYEA_OK;
    free(n->parameters); free(n->gradient);
    for (int k = 0; k < MYEA_STATE_KINDS; ++k) free(n->opt[k]);
    free(n->masks); free(n->zoneout);
    for (size_t li = 0; li < n->d.n_layers; ++li) {
        olayer *o = &n->L[li];
        free(o->summations); free(o->values); free(o->hats); free(o->normalizes);
        free(o->neuron_errors); free(o->af_errors); free(o->norm_errors);
        free(o->means); free(o->variances); free(o->means_averages); free(o->variances_averages);
        free(o->r_corrections); free(o->d_corrections); free(o->derivatives_means); free(o->derivatives_variances);
        free(o->pool_index); free(o->pre_afs); free(o->dafs); free(o->noise);
        free(o->unit_af); free(o->unit_steep);
        if (o->lstm) {
            for (int dir = 0; dir < 2; ++dir) {
                olstm *q = &o->lstm[dir];
                float *all[] = {q->sum_in_z, q->sum_rec_z, q->sum_z, q->z, q->c, q->ca, q->dz, q->dc, q->sum_in_i, q->sum_in_f, q->sum_in_o, q->sum_rec_i,
                                q->sum_rec_f, q->sum_rec_o, q->sum_i, q->sum_f, q->sum_o, q->gi, q->gf, q->go, q->di, q->df, q->dgo};
                for (size_t a = 0; a < sizeof(all) / sizeof(all[0]); ++a) free(all[a]);
                if (q->norm) {
                    for (int g = 0; g < 9; ++g) {
                        obn *bn = &q->nrm[g];
                        float *bns[] = {bn->means, bn->variances, bn->means_averages, bn->variances_averages, bn->r_corrections, bn->d_corrections,
                                        bn->derivatives_means, bn->derivatives_variances, bn->hats, bn->normalizes};
                        for (size_t a = 0; a < sizeof(bns) / sizeof(bns[0]); ++a) free(bns[a]);
                    }
                    float *ds[] = {q->dz_in, q->dz_rec, q->di_in, q->di_rec, q->df_in, q->df_rec, q->do_in, q->do_rec};
                    for (size_t a = 0; a < 8; ++a) free(ds[a]);
                }
                if (q->h != o->values) free(q->h);
                if (q->dh != o->af_errors) free(q->dh);
            }
            free(o->lstm);
        }
    }
    free(n);
    return MYEA_OK;
}

int myea_oracle_set_hyper(myea_oracle_net *n, const myea_hyper *h) { if (!n || !h) return MYEA_E_INVALID; n->h = *h; return MYEA_OK; }
int myea_oracle_get_hyper(myea_oracle_net *n, myea_hyper *h) { if (!n || !h) return MYEA_E_INVALID; *h = n->h; return MYEA_OK; }
int myea_oracle_set_state_propagation(myea_oracle_net *n, uint32_t s) { if (!n) return MYEA_E_INVALID; n->state = s; return MYEA_OK; }
/* AF_unit::ptr_type_activation_function / ptr_activation_steepness as per-unit arrays (NNH/Data.hpp, struct AF_unit) */
int myea_oracle_set_unit_activations(myea_oracle_net *n, size_t li, const uint32_t *types, const float *steep, size_t count)
{
    if (!n || li == 0 || li >= n->d.n_layers || !is_dense(&n->d.layers[li])) return MYEA_E_INVALID;
    olayer *o = &n->L[li];
    if (((types || steep) && count != o->AH) || n->d.layers[li].type_activation_function == MYEA_AF_SOFTMAX) return MYEA_E_INVALID;
    free(o->unit_af); free(o->unit_steep); o->unit_af = NULL; o->unit_steep = NULL;
    if (types) {
        for (size_t j = 0; j < count; ++j) if (types[j] == MYEA_AF_NONE || types[j] >= MYEA_AF_LENGTH || types[j] == MYEA_AF_SOFTMAX) return MYEA_E_INVALID;
        o->unit_af = (uint32_t *)malloc(count * sizeof(uint32_t)); memcpy(o->unit_af, types, count * sizeof(uint32_t));
    }
    if (steep) { o->unit_steep = (float *)malloc(count * sizeof(float)); memcpy(o->unit_steep, steep, count * sizeof(float)); }
    return MYEA_OK;
}
int myea_oracle_set_threads(myea_oracle_net *n, int t) { if (!n || t < 1) return MYEA_E_INVALID; n->threads = t; return MYEA_OK; }
float *myea_oracle_parameters(myea_oracle_net *n) { return n->parameters; }
float *myea_oracle_gradient(myea_oracle_net *n) { return n->gradient; }
float *myea_oracle_optimizer_state(myea_oracle_net *n, int k) { return (k >= 0 && k < MYEA_STATE_KINDS) ? n->opt[k] : NULL; }
float *myea_oracle_dropout_noise(myea_oracle_net *n, size_t li, size_t *count)
{
    if (!n || li >= n->d.n_layers || !n->L[li].noise) { if (count) *count = 0; return NULL; }
    if (n->d.layers[li].type_layer == MYEA_LAYER_RESIDUAL) { if (count) *count = (size_t)n->d.number_recurrent_depth * n->d.batch_size * (1 + 2 * n->L[li].NH); return n->L[li].noise; }
    if (count) *count = (size_t)n->d.number_recurrent_depth * n->d.batch_size * n->L[li].AH;
    return n->L[li].noise;
}
uint8_t *myea_oracle_zoneout_masks(myea_oracle_net *n, size_t *count) { if (count) *count = n->zoneout_count; return n->zoneout; }
uint8_t *myea_oracle_masks(myea_oracle_net *n) { return n->masks; }

/* Clear_Optimizer NN/Train.cpp:128-263: a switch on the current optimizer - only ITS state is cleared (:134-258) - then
 * optimizer_time_step = 0, epoch_time_step = 1 for all (:260-261) */
static void clear_optimizer(myea_oracle_net *n)
{
    size_t P = n->d.total_parameters, bytes = P * sizeof(float);
    switch (n->h.type_optimizer_function) {
    case MYEA_OPTIMIZER_NONE: break;
    case MYEA_OPTIMIZER_GD:                                    /* :136-143 */
        if (n->h.learning_momentum != 0.f) memset(n->opt[MYEA_STATE_PREVIOUS_DELTA], 0, bytes);
        break;
    case MYEA_OPTIMIZER_IRPROP_PLUS:                           /* :166-198 */
        n->h.loss_rprop = FLT_MAX;
        n->h.previous_loss_rprop = FLT_MAX;
        memset(n->opt[MYEA_STATE_PREVIOUS_DERIVATIVES], 0, bytes);
        for (size_t i = 0; i < P; ++i) n->opt[MYEA_STATE_PREVIOUS_STEPS][i] = n->h.rprop_delta_zero;
        memset(n->opt[MYEA_STATE_PREVIOUS_DELTA], 0, bytes);
        break;
    case MYEA_OPTIMIZER_AMSBOUND:
    case MYEA_OPTIMIZER_AMSGRAD:                               /* :201-223 */
        memset(n->opt[MYEA_STATE_FIRST_MOMENT], 0, bytes);
        memset(n->opt[MYEA_STATE_SECOND_MOMENT], 0, bytes);
        memset(n->opt[MYEA_STATE_SECOND_MOMENT_HAT], 0, bytes);
        break;
    case MYEA_OPTIMIZER_ADABOUND:
    case MYEA_OPTIMIZER_ADAM:                                  /* :224-240 */
        memset(n->opt[MYEA_STATE_FIRST_MOMENT], 0, bytes);
        memset(n->opt[MYEA_STATE_SECOND_MOMENT], 0, bytes);
        break;
    case MYEA_OPTIMIZER_NOSADAM:                               /* :241-257 */
        memset(n->opt[MYEA_STATE_FIRST_MOMENT], 0, bytes);
        memset(n->opt[MYEA_STATE_SECOND_MOMENT], 0, bytes);
        n->h.adam_previous_beta2 = 0.f;
        break;
    default: break;
    }
    n->h.optimizer_time_step = 0.f;
    n->h.epoch_time_step = 1.f;
}

/* Clear_Training_Arrays NN/Train.cpp:93-126 */
int myea_oracle_clear_training_arrays(myea_oracle_net *n)
{
    size_t P = n->d.total_parameters;
    memset(n->gradient, 0, P * sizeof(float));
    clear_optimizer(n);
    return MYEA_OK;
}

/* ------------------------------------------------------------------------------------------- */
/* forward pieces */

/* Forward_Pass__FC: NN/Neural_Network__Forward_Pass__OpenMP.cpp:4517-4557 */
static void fwd_fc(myea_oracle_net *n, size_t t, size_t B, size_t In, size_t Out, const float *x, const float *w, float *y)
{
    size_t Bmax = n->d.batch_size;
    const float *xt = x + Bmax * In * t;
    float *yt = y + Bmax * Out * t;
    long b;
#pragma omp parallel for schedule(static) num_threads(n->threads)
    for (b = 0; b < (long)B; ++b) {
        const float *xi = xt + (size_t)b * In;
        float *yo = yt + (size_t)b * Out;
        for (size_t o = 0; o < Out; ++o) {
            const float *wr = w + o * In;
            float s = 0.f;
            for (size_t i = 0; i < In; ++i) s += xi[i] * wr[i];
            yo[o] = s;
        }
    }
}

/* Forward_Pass__Bias: NN/Neural_Network__Forward_Pass__OpenMP.cpp:4494-4515 */
static void fwd_bias(myea_oracle_net *n, size_t t, size_t B, size_t Out, const float *bias, float *y)
{
    float *yt = y + n->d.batch_size * Out * t;
    for (size_t b = 0; b < B; ++b)
        for (size_t o = 0; o < Out; ++o) yt[b * Out + o] += bias[o];
}

/* Forward_Pass__Batch_Normalization__Training: NN/Neural_Network__Forward_Pass__OpenMP.cpp:4591-4701
 * Forward_Pass__Batch_Renormalization__Training: :4703-4837.
 * `variances` receives sqrt(var + eps) (:4675). */
static void fwd_bn_training(myea_oracle_net *n, int renorm, size_t t, size_t B, size_t H, const float *x,
                            const float *scale, const float *shift, olayer *o)
{
    size_t Bmax = n->d.batch_size;
    const float *xt = x + Bmax * H * t;
    float *mean = o->means + t * H, *var = o->variances + t * H;
    float *mavg = o->means_averages + t * H, *vavg = o->variances_averages + t * H;
    float *rc = o->r_corrections + t * H, *dc = o->d_corrections + t * H;
    float *hat = o->hats + Bmax * H * t, *nor = o->normalizes + Bmax * H * t;
    float bscale = 1.f / (float)B, eps = n->h.normalization_epsilon, mom = n->h.normalization_momentum_average;
    float rmax = n->h.batch_renormalization_r_correction_maximum, dmax = n->h.batch_renormalization_d_correction_maximum;
    for (size_t j = 0; j < H; ++j) { mean[j] = 0.f; var[j] = 0.f; } /* MEMSET at the start of the pass, :54-66 */
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) { float s = xt[b * H + j]; mean[j] += s; var[j] += s * s; }
    for (size_t j = 0; j < H; ++j) {
        mean[j] *= bscale;
        mavg[j] += mom * (mean[j] - mavg[j]);
        var[j] = sqrtf(var[j] * bscale - mean[j] * mean[j] + eps);
        vavg[j] += mom * (var[j] - vavg[j]);
        if (renorm) {
            float g = var[j] / vavg[j], lo = 1.f / rmax;
            rc[j] = g < lo ? lo : (g > rmax ? rmax : g);
            float dd = (mean[j] - mavg[j]) / vavg[j];
            dc[j] = dd < -dmax ? -dmax : (dd > dmax ? dmax : dd);
        }
    }
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) {
            float s = xt[b * H + j];
            if (renorm) s = (s - mean[j]) / var[j] * rc[j] + dc[j];
            else s = (s - mean[j]) / var[j];
            hat[b * H + j] = s;
            nor[b * H + j] = scale[j] * s + shift[j];
        }
}

/* Forward_Pass__Batch_Normalization__Inference: NN/Neural_Network__Forward_Pass__OpenMP.cpp:4559-4589 */
static void fwd_bn_inference(myea_oracle_net *n, size_t t, size_t B, size_t H, const float *x, const float *scale, const float *shift, olayer *o)
{
    size_t Bmax = n->d.batch_size;
    const float *xt = x + Bmax * H * t;
    float *nor = o->normalizes + Bmax * H * t;
    const float *mavg = o->means_averages + t * H, *vavg = o->variances_averages + t * H;
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) nor[b * H + j] = scale[j] * ((xt[b * H + j] - mavg[j]) / vavg[j]) + shift[j];
}

/* Forward_Pass__FC_AF: :4839-4868; Forward_Pass__FC_AF__Softmax: :4870-4905 */
static void fwd_af(myea_oracle_net *n, size_t t, size_t B, size_t H, uint32_t type, const uint32_t *unit_type, const float *x, float *y)
{
    size_t off = n->d.batch_size * H * t;
    for (size_t b = 0; b < B; ++b) {
        const float *xi = x + off + b * H;
        float *yo = y + off + b * H;
        if (type == MYEA_AF_SOFTMAX) {
            float mx = -FLT_MAX, sum = 0.f;
            for (size_t j = 0; j < H; ++j) mx = mx > xi[j] ? mx : xi[j];
            for (size_t j = 0; j < H; ++j) sum += yo[j] = expf(xi[j] - mx);
            sum = 1.f / sum;
            for (size_t j = 0; j < H; ++j) yo[j] *= sum;
        } else {
            for (size_t j = 0; j < H; ++j) yo[j] = myea_oracle_activation(unit_type ? unit_type[j] : type, xi[j]);
        }
    }
}

/* Forward_Pass__Dropout__Bernoulli__{Training,Inverted,Inference}: :4907-4990.
 * mask is per (t, unit), shared by every example. */
static void fwd_dropout(myea_oracle_net *n, const myea_layer_desc *l, size_t t, size_t B, size_t H, float *v)
{
    size_t off = n->d.batch_size * H * t;
    const float *li_noise = n->L[l - n->d.layers].noise;
    const uint8_t *m = n->masks + l->first_mask_index + t * H;
    if (n->state == MYEA_STATE_TRAINING) {
        if (l->type_dropout == MYEA_DROPOUT_BERNOULLI) {
            for (size_t b = 0; b < B; ++b)
                for (size_t j = 0; j < H; ++j) if (!m[j]) v[off + b * H + j] = 0.f;
        } else if (l->type_dropout == MYEA_DROPOUT_BERNOULLI_INVERTED) {
            float inv = l->dropout_values[0] == 0.f ? 0.f : 1.f / l->dropout_values[0];
            for (size_t b = 0; b < B; ++b)
                for (size_t j = 0; j < H; ++j) { if (m[j]) v[off + b * H + j] *= inv; else v[off + b * H + j] = 0.f; }
        }
    } else if (l->type_dropout == MYEA_DROPOUT_BERNOULLI) {
        for (size_t b = 0; b < B; ++b)
            for (size_t j = 0; j < H; ++j) v[off + b * H + j] *= l->dropout_values[0];
    }
    /* Forward_Pass__Dropout__Gaussian (NN/Neural_Network__Forward_Pass__Loop.cpp:4993-5014): v *= N(1, dropout_values[0]);
     * Forward_Pass__Dropout__Uout (:5047-5068): v += v * U(-dropout_values[0], +dropout_values[0]); strictly in the training
     * state, one draw per (example, unit), example-major - here read from the supplied tensor */
    if (n->state == MYEA_STATE_TRAINING && li_noise) {
        if (l->type_dropout == MYEA_DROPOUT_GAUSSIAN) {
            for (size_t b = 0; b < B; ++b)
                for (size_t j = 0; j < H; ++j) v[off + b * H + j] *= li_noise[off + b * H + j];
        } else if (l->type_dropout == MYEA_DROPOUT_UOUT) {
            for (size_t b = 0; b < B; ++b)
                for (size_t j = 0; j < H; ++j) v[off + b * H + j] += v[off + b * H + j] * li_noise[off + b * H + j];
        }
    }
}

/* Sparse_K_Filter (NN/Neural_Network__K_Sparse.cpp:268-339): per example, the k largest values of the row stay where they
 * are and the others become 0.  The reference keeps a sorted array of (index, value) pairs seeded with the first k entries
 * and lets a later entry replace the smallest pair only when it is strictly greater; which of several EQUAL smallest pairs
 * goes is left to std::sort's unspecified order of equal keys.  Restated with that choice fixed: among equal values the
 * lower index stays.  Rows without equal values at the cut are unaffected by the choice. */
static void fwd_k_sparse(myea_oracle_net *n, size_t t, size_t B, size_t H, size_t k, float *v)
{
    if (k >= H) return;
    size_t off = n->d.batch_size * H * t;
    size_t *idx = (size_t *)malloc((k ? k : 1) * sizeof(size_t));
    float *val = (float *)malloc((k ? k : 1) * sizeof(float));
    for (size_t b = 0; b < B; ++b) {
        float *row = v + off + b * H;
        size_t kept = 0;
        /* pairs ascending by (value, then index descending): slot 0 is the one to go - the smallest value, and among equal
         * values the highest index */
        for (size_t j = 0; j < H; ++j) {
            if (kept == k) {
                if (!(val[0] < row[j])) continue;   /* strictly greater only */
                /* drop slot 0 */
                for (size_t s = 1; s < kept; ++s) { val[s - 1] = val[s]; idx[s - 1] = idx[s]; }
                --kept;
            }
            /* insert (j, row[j]); j is the highest index so far, so among equal values it goes in front */
            size_t at = 0;
            while (at < kept && val[at] < row[j]) ++at;
            for (size_t s = kept; s > at; --s) { val[s] = val[s - 1]; idx[s] = idx[s - 1]; }
            val[at] = row[j]; idx[at] = j;
            ++kept;
        }
        memset(row, 0, H * sizeof(float));
        for (size_t s = 0; s < kept; ++s) row[idx[s]] = val[s];
    }
    free(idx); free(val);
}

/* Forward_Pass__FC_Ind_RNN (NN/Neural_Network__Recurrent_Forward_Pass__Loop.cpp:813-866): pre_AF[t] = input[t] + u * AF[t-1],
 * a plain copy at the first time step.  AF[t-1] is what the previous time step left in the array: after an un-normalised
 * layer's dropout, which works in place on it. */
static void fwd_ind_rnn(myea_oracle_net *n, size_t t, size_t B, size_t H, const float *u, const float *afs, const float *in, float *pre_afs)
{
    size_t Bmax = n->d.batch_size, off = Bmax * H * t, prev = t ? Bmax * H * (t - 1) : 0;
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) {
            size_t k = off + b * H + j;
            pre_afs[k] = t ? in[k] + u[j] * afs[prev + b * H + j] : in[k];
        }
}

/* Forward_Pass__FC (layer driver): NN/Neural_Network__Forward_Pass__OpenMP.cpp:256-698 (the serial build's
 * NN/Neural_Network__Forward_Pass__Loop.cpp:350-790 carries the independently recurrent branch).
 * order: GEMM -> bias -> [BN before] -> [+ u * AF[t-1]] -> activation / softmax -> [BN after] -> dropout. */
static void fwd_fc_layer(myea_oracle_net *n, size_t li, size_t t, size_t B)
{
    const myea_layer_desc *l = &n->d.layers[li];
    olayer *o = &n->L[li];
    size_t In = o->In, H = o->H;
    const float *x = layer_outputs(n, o->prev);
    int training = n->state >= MYEA_STATE_TRAINING;
    int renorm = l->type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
    fwd_fc(n, t, B, In, H, x, n->parameters + l->first_connection_index, o->summations);
    if (layer_uses_bias(l)) fwd_bias(n, t, B, H, n->parameters + l->first_bias_connection_index, o->summations);
    const float *cur = o->summations;
    if (layer_uses_norm(l) && l->use_layer_normalization_before_activation) {
        if (training) fwd_bn_training(n, renorm, t, B, H, cur, scale_ptr(n, n->parameters, li), shift_ptr(n, n->parameters, li), o);
        else fwd_bn_inference(n, t, B, H, cur, scale_ptr(n, n->parameters, li), shift_ptr(n, n->parameters, li), o);
        cur = o->normalizes;
    }
    if (is_ind_rnn(l)) {
        fwd_ind_rnn(n, t, B, H, n->parameters + l->first_connection_index + H * In, o->values, cur, o->pre_afs);
        cur = o->pre_afs;
    }
    fwd_af(n, t, B, H, l->type_activation_function, o->unit_af, cur, o->values);
    float *out = o->values;
    if (layer_uses_norm(l) && !l->use_layer_normalization_before_activation) {
        if (training) fwd_bn_training(n, renorm, t, B, H, o->values, scale_ptr(n, n->parameters, li), shift_ptr(n, n->parameters, li), o);
        else fwd_bn_inference(n, t, B, H, o->values, scale_ptr(n, n->parameters, li), shift_ptr(n, n->parameters, li), o);
        out = o->normalizes;
    }
    fwd_dropout(n, l, t, B, H, out);
    /* k-Sparse, after the dropout (NN/Neural_Network__Forward_Pass__Loop.cpp:752-790): k values stay strictly in the
     * training state, size_t(alpha * k) otherwise */
    if (l->k_sparsity != 0)
        fwd_k_sparse(n, t, B, H, n->state == MYEA_STATE_TRAINING ? (size_t)l->k_sparsity : (size_t)(l->alpha_sparsity * (float)l->k_sparsity), out);
}

static void fwd_pooling(myea_oracle_net *n, size_t li, size_t t, size_t B);

/* Forward_Pass__Residual__FC: NN/Neural_Network__Forward_Pass__OpenMP.cpp:4039-4433.  Pre-activation order on the
 * layer's INPUT (fan-in wide): [BN] -> (not for the block's first layer: activation -> dropout) -> weights -> bias.
 * The layer's output is its summation. */
static void fwd_residual_fc_layer(myea_oracle_net *n, size_t li, size_t t, size_t B)
{
    const myea_layer_desc *l = &n->d.layers[li];
    olayer *o = &n->L[li];
    size_t In = o->In, H = o->H;
    const float *cur = layer_outputs(n, o->prev);
    int training = n->state >= MYEA_STATE_TRAINING;
    int renorm = l->type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
    if (layer_uses_norm(l)) {
        if (training) fwd_bn_training(n, renorm, t, B, In, cur, scale_ptr(n, n->parameters, li), shift_ptr(n, n->parameters, li), o);
        else fwd_bn_inference(n, t, B, In, cur, scale_ptr(n, n->parameters, li), shift_ptr(n, n->parameters, li), o);
        cur = o->normalizes;
    }
    if (o->group == 2) {
        if (is_ind_rnn(l)) {   /* the recurrence sits on the member's input side too (:4108-4150): self weights behind the [H][In] matrix */
            fwd_ind_rnn(n, t, B, In, n->parameters + l->first_connection_index + H * In, o->values, cur, o->pre_afs);
            cur = o->pre_afs;
        }
        fwd_af(n, t, B, In, l->type_activation_function, o->unit_af, cur, o->values);
        fwd_dropout(n, l, t, B, In, o->values);   /* Bernoulli (training masks, inference scaling), Gaussian, Uout: :4197-4232, :4253-4262 */
        if (l->k_sparsity != 0)                   /* :4234-4245, :4264-4274 */
            fwd_k_sparse(n, t, B, In, n->state == MYEA_STATE_TRAINING ? (size_t)l->k_sparsity : (size_t)(l->alpha_sparsity * (float)l->k_sparsity), o->values);
        cur = o->values;
    }
    fwd_fc(n, t, B, In, H, cur, n->parameters + l->first_connection_index, o->summations);
    if (layer_uses_bias(l)) fwd_bias(n, t, B, H, n->parameters + l->first_bias_connection_index, o->summations);
}

/* Forward_Pass__Residual: :3861-3997 (block members, then [block-level BN] on the last member's output, then the
 * shortcut); Forward_Pass__Zero_Padded_Identity: :5158-5240 (A = shortcut source, B = block output; the narrower one is
 * added into the wider one at offset `padding`). */
/* With a recurrent depth T > 1 every member and the shortcut run time step by time step on the [T][Bmax][width] tensors
 * (Recurrent__Forward_Pass__Residual / __Residual__FC / __Zero_Padded_Identity,
 * NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:563-817: loops over the time steps around the same functions). */
static void fwd_lstm_layer(myea_oracle_net *n, size_t li, size_t B);

/* the members, one after the other, each over all of its time steps (Recurrent__Forward_Pass__Residual__Layer,
 * NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:711-771; feed-forward: Forward_Pass__Residual__Layer, :3999-4036) */
static void fwd_residual_members(myea_oracle_net *n, size_t ri, size_t B)
{
    size_t last = ri + n->d.layers[ri].block_depth, T = n->d.number_recurrent_depth;
    for (size_t li = ri + 1; li <= last; ++li) {
        const myea_layer_desc *l = &n->d.layers[li];
        if (l->type_layer == MYEA_LAYER_LSTM) fwd_lstm_layer(n, li, B);
        else for (size_t t = 0; t < T; ++t) {
            if (is_pooling(l)) fwd_pooling(n, li, t, B);
            else fwd_residual_fc_layer(n, li, t, B);
        }
    }
}

static void fwd_residual_block(myea_oracle_net *n, size_t ri, size_t t, size_t B)
{
    const myea_layer_desc *r = &n->d.layers[ri];
    olayer *o = &n->L[ri];
    size_t last = ri + r->block_depth, Bmax = n->d.batch_size;
    float *blk = layer_outputs(n, last);
    size_t nb = n->L[last].H, na = n->L[o->prev].H;
    if (layer_uses_norm(r)) {
        int renorm = r->type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
        if (n->state >= MYEA_STATE_TRAINING) fwd_bn_training(n, renorm, t, B, nb, blk, scale_ptr(n, n->parameters, ri), shift_ptr(n, n->parameters, ri), o);
        else fwd_bn_inference(n, t, B, nb, blk, scale_ptr(n, n->parameters, ri), shift_ptr(n, n->parameters, ri), o);
        blk = o->normalizes;
    }
    blk += t * Bmax * nb;   /* the time step's rows, from here on */
    /* ShakeDrop on the block's output, in place (Forward_Pass__Residual__Block, NN/Neural_Network__Forward_Pass__Loop.cpp:4053-4078;
     * Forward_Pass__Dropout__ShakeDrop :5016-5045): strictly in the training state an example is perturbed with probability
     * dropout_values[0], each of its values then times its own U(-1, 1) draw; otherwise every value times 1 - dropout_values[0].
     * Draws as supplied: [mask per example][forward draws][backward draws]. */
    if (r->type_dropout == MYEA_DROPOUT_SHAKEDROP) {
        /* one mask per (time step, example), one draw per (time step, example, value): [T][Bmax] masks, then the forward
         * draws [T][Bmax][width], then the backward draws (Recurrent__Forward_Pass__Dropout__ShakeDrop,
         * NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:367-386, indexes the mask with batch_size x time step + example) */
        const size_t T = n->d.number_recurrent_depth;
        const float *mask = o->noise + t * Bmax, *alpha = o->noise + T * Bmax + t * Bmax * nb;
        for (size_t b = 0; b < B; ++b)
            for (size_t j = 0; j < nb; ++j) {
                if (n->state == MYEA_STATE_TRAINING) { if (mask[b] != 0.f) blk[b * nb + j] *= alpha[b * nb + j]; }
                else blk[b * nb + j] *= 1.f - r->dropout_values[0];
            }
    }
    const float *a = layer_outputs(n, o->prev) + t * Bmax * na;
    float *values = o->values + t * Bmax * o->H;
    for (size_t b = 0; b < B; ++b) {
        const float *ar = a + b * na, *br = blk + b * nb;
        if (o->pad == 0) {
            float *y = values + b * na;
            for (size_t j = 0; j < na; ++j) y[j] = ar[j] + br[j];
        } else if (na > nb) {
            float *y = values + b * na;
            for (size_t j = 0; j < na; ++j) y[j] = ar[j];
            for (size_t j = 0; j < nb; ++j) y[j + o->pad] += br[j];
        } else {
            float *y = values + b * nb;
            for (size_t j = 0; j < nb; ++j) y[j] = br[j];
            for (size_t j = 0; j < na; ++j) y[j + o->pad] += ar[j];
        }
    }
}

/* ------------------------------------------------------------------------------------------- */
/* The same normalisation on one group of an LSTM layer's normalised units: training (:4591-4701 / :4703-4837), inference
 * (:4559-4589), and the backward pass WITHOUT a shift gradient that the LSTM path calls
 * (NN/Neural_Network__Backward_Pass__OpenMP.cpp:1469-1584, renormalised :1711-1829; dy and dx may be the same array). */
static void lstm_bn_forward(myea_oracle_net *n, int renorm, obn *bn, size_t t, size_t B, const float *x)
{
    size_t Bmax = n->d.batch_size, H = bn->H, off = Bmax * H * t;
    const float *scale = n->parameters + bn->param, *shift = scale + n->d.total_normalized_units;
    const float *xt = x + off;
    float *hat = bn->hats + off, *nor = bn->normalizes + off;
    float *mavg = bn->means_averages + t * H, *vavg = bn->variances_averages + t * H;
    if (n->state < MYEA_STATE_TRAINING) {
        for (size_t b = 0; b < B; ++b)
            for (size_t j = 0; j < H; ++j) nor[b * H + j] = scale[j] * ((xt[b * H + j] - mavg[j]) / vavg[j]) + shift[j];
        return;
    }
    float *mean = bn->means + t * H, *var = bn->variances + t * H, *rc = bn->r_corrections + t * H, *dc = bn->d_corrections + t * H;
    float bscale = 1.f / (float)B, eps = n->h.normalization_epsilon, mom = n->h.normalization_momentum_average;
    float rmax = n->h.batch_renormalization_r_correction_maximum, dmax = n->h.batch_renormalization_d_correction_maximum;
    for (size_t j = 0; j < H; ++j) { mean[j] = 0.f; var[j] = 0.f; }
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) { float v = xt[b * H + j]; mean[j] += v; var[j] += v * v; }
    for (size_t j = 0; j < H; ++j) {
        mean[j] *= bscale;
        mavg[j] += mom * (mean[j] - mavg[j]);
        var[j] = sqrtf(var[j] * bscale - mean[j] * mean[j] + eps);
        vavg[j] += mom * (var[j] - vavg[j]);
        if (renorm) {
            float g = var[j] / vavg[j], lo = 1.f / rmax;
            rc[j] = g < lo ? lo : (g > rmax ? rmax : g);
            float dd = (mean[j] - mavg[j]) / vavg[j];
            dc[j] = dd < -dmax ? -dmax : (dd > dmax ? dmax : dd);
        }
    }
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) {
            float v = xt[b * H + j];
            if (renorm) v = (v - mean[j]) / var[j] * rc[j] + dc[j];
            else v = (v - mean[j]) / var[j];
            hat[b * H + j] = v;
            nor[b * H + j] = scale[j] * v + shift[j];
        }
}

static void lstm_bn_backward(myea_oracle_net *n, int renorm, obn *bn, size_t t, size_t B, const float *x, float *d)
{
    size_t Bmax = n->d.batch_size, H = bn->H, off = Bmax * H * t;
    const float *mean = bn->means + t * H, *var = bn->variances + t * H, *rc = bn->r_corrections + t * H;
    const float *scale = n->parameters + bn->param;
    float *dscale = n->gradient + bn->param;
    float *dmean = bn->derivatives_means + t * H, *dvar = bn->derivatives_variances + t * H;
    float bscale = 1.f / (float)B;
    for (size_t j = 0; j < H; ++j) { dmean[j] = 0.f; dvar[j] = 0.f; }
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) {
            size_t k = off + b * H + j;
            float e = d[k], vb = var[j], r = renorm ? rc[j] : 1.f;
            dscale[j] += e * bn->hats[k];
            e *= scale[j];
            dmean[j] += e * (-r / vb);
            dvar[j] += e * (x[k] - mean[j]) * (-r / (vb * vb));
            d[k] = e;
        }
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) {
            size_t k = off + b * H + j;
            float e = d[k], vb = var[j], r = renorm ? rc[j] : 1.f;
            e *= r / vb;
            e += dvar[j] * ((x[k] - mean[j]) / ((float)B * vb));
            e += dmean[j] * bscale;
            d[k] = e;
        }
}

/* ------------------------------------------------------------------------------------------- */
/* LSTM with peepholes (one direction, time ascending) */

/* parameter offsets inside the layer's slice, NN/Neural_Network__Prepare_Connections.cpp:82-222: per block
 * [z_in(In) | z_rec(C)] x cells, i_in, f_in, o_in (In each), i_rec, f_rec, o_rec (C each), peep_i, peep_f, peep_o (cpb each) */
static size_t lstm_block_base(const myea_layer_desc *l, const olstm *q, size_t k) { (void)l; return q->base + k * q->per_block; }
static size_t lstm_z_in(const myea_layer_desc *l, const olstm *q, size_t k, size_t j) { return lstm_block_base(l, q, k) + j * (q->In + q->C); }
static size_t lstm_z_rec(const myea_layer_desc *l, const olstm *q, size_t k, size_t j) { return lstm_z_in(l, q, k, j) + q->In; }
static size_t lstm_gate_in(const myea_layer_desc *l, const olstm *q, size_t k, int g) { return lstm_block_base(l, q, k) + q->cpb * (q->In + q->C) + (size_t)g * q->In; }
static size_t lstm_gate_rec(const myea_layer_desc *l, const olstm *q, size_t k, int g) { return lstm_gate_in(l, q, k, 3) + (size_t)g * q->C; }
static size_t lstm_peep(const myea_layer_desc *l, const olstm *q, size_t k, int g) { return lstm_gate_rec(l, q, k, 3) + (size_t)g * q->cpb; }

static float sigmoid_f(float s) { return 1.f / (1.f + expf(-s)); }
static float tanh_f(float s) { return 2.f / (1.f + expf(-2.f * s)) - 1.f; }

/* Forward_Pass__LSTM (NN/Neural_Network__Forward_Pass__OpenMP.cpp:1769-2340), training and inference alike without
 * normalisation / zoneout: Gates_CIFO (NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:859-1040) ->
 * Gates_CIF_AF_State (:1042-1191) -> States_AF (:1547-1582) -> Output (:1351-1418).
 * First step: no recurrent sums, no forget gate, no input-gate peephole, c = i * z; the output gate peeps at c[t].
 * Bias vectors sit at first_bias_connection_index + {0, C, C + K, C + 2K} (the field as Prepare__Bias__LSTM leaves it). */
static void fwd_lstm_step(myea_oracle_net *n, size_t li, int dir, size_t t, size_t B)
{
    const myea_layer_desc *l = &n->d.layers[li];
    olayer *o = &n->L[li];
    olstm *q = &o->lstm[dir];
    size_t Bmax = n->d.batch_size, K = q->K, C = q->C, cpb = q->cpb, In = q->In;
    const float *x = layer_outputs(n, n->L[li].prev), *w = n->parameters;
    const float *bz = w + q->bias, *bi = bz + C, *bf = bi + K, *bo = bf + K;
    /* the step processed before this one: t - 1, or t + 1 for the direction that walks time backwards
     * (tmp_time_step_reverse_direction, NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:456-461) */
    size_t tp = q->reverse ? t + 1 : t - 1;
    int first = q->reverse ? t == n->d.number_recurrent_depth - 1 : t == 0;
    /* strictly in the training state (NN/Neural_Network__Forward_Pass__Loop.cpp:2088-2092) */
    int zone = l->type_dropout == MYEA_DROPOUT_ZONEOUT && n->state == MYEA_STATE_TRAINING;
    long b;
#pragma omp parallel for schedule(static) num_threads(n->threads)
    for (b = 0; b < (long)B; ++b) {
        size_t kb = (size_t)b * K + Bmax * K * t, cb = (size_t)b * C + Bmax * C * t, cp = (size_t)b * C + Bmax * C * tp;
        const float *xi = x + (size_t)b * In + Bmax * In * t;
        const float *hp = first ? NULL : q->h + cp;
        for (size_t k = 0; k < K; ++k) {
            for (size_t j = 0; j < cpb; ++j) {
                size_t c = k * cpb + j;
                const float *wi = w + lstm_z_in(l, q, k, j), *wr = w + lstm_z_rec(l, q, k, j);
                float s = 0.f;
                for (size_t a = 0; a < In; ++a) s += xi[a] * wi[a];
                q->sum_in_z[cb + c] = s;
                if (!first) { s = 0.f; for (size_t a = 0; a < C; ++a) s += hp[a] * wr[a]; q->sum_rec_z[cb + c] = s; }
            }
            float si = 0.f, sf = 0.f, so = 0.f;
            const float *wi = w + lstm_gate_in(l, q, k, 0), *wf = w + lstm_gate_in(l, q, k, 1), *wo = w + lstm_gate_in(l, q, k, 2);
            for (size_t a = 0; a < In; ++a) { si += xi[a] * wi[a]; sf += xi[a] * wf[a]; so += xi[a] * wo[a]; }
            q->sum_in_i[kb + k] = si; q->sum_in_f[kb + k] = sf; q->sum_in_o[kb + k] = so;
            if (!first) {
                si = sf = so = 0.f;
                wi = w + lstm_gate_rec(l, q, k, 0); wf = w + lstm_gate_rec(l, q, k, 1); wo = w + lstm_gate_rec(l, q, k, 2);
                for (size_t a = 0; a < C; ++a) { si += hp[a] * wi[a]; sf += hp[a] * wf[a]; so += hp[a] * wo[a]; }
                q->sum_rec_i[kb + k] = si; q->sum_rec_f[kb + k] = sf; q->sum_rec_o[kb + k] = so;
            }
        }
        /* Gates_CIF_AF_State */
        for (size_t k = 0; k < K; ++k) {
            const float *pi = w + lstm_peep(l, q, k, 0), *pf = w + lstm_peep(l, q, k, 1);
            if (!first) {
                float si = q->sum_in_i[kb + k] + q->sum_rec_i[kb + k] + bi[k];
                float sf = q->sum_in_f[kb + k] + q->sum_rec_f[kb + k] + bf[k];
                for (size_t j = 0; j < cpb; ++j) { si += q->c[cp + k * cpb + j] * pi[j]; sf += q->c[cp + k * cpb + j] * pf[j]; }
                q->sum_i[kb + k] = si; q->sum_f[kb + k] = sf;
                q->gi[kb + k] = sigmoid_f(si); q->gf[kb + k] = sigmoid_f(sf);
            } else {
                float si = q->sum_in_i[kb + k] + bi[k];
                q->sum_i[kb + k] = si;
                q->gi[kb + k] = sigmoid_f(si);
            }
            for (size_t j = 0; j < cpb; ++j) {
                size_t c = k * cpb + j;
                float sz = first ? q->sum_in_z[cb + c] + bz[c] : q->sum_in_z[cb + c] + q->sum_rec_z[cb + c] + bz[c];
                q->sum_z[cb + c] = sz;
                q->z[cb + c] = tanh_f(sz);
                q->c[cb + c] = first ? q->z[cb + c] * q->gi[kb + k] : q->z[cb + c] * q->gi[kb + k] + q->gf[kb + k] * q->c[cp + c];
                /* zoneout of the cell state (Forward_Pass__LSTM__Gates_CIF_AF_State__Zoneout, :1285-1288, :1331-1334) */
                if (zone && !q->zone_state[t * q->zone_stride + c]) q->c[cb + c] = first ? 0.f : q->c[cp + c];
            }
        }
        /* States_AF */
        for (size_t c = 0; c < C; ++c) q->ca[cb + c] = tanh_f(q->c[cb + c]);
        /* Output: the recurrent sum of the first step is never written by the reference and stays 0 */
        for (size_t k = 0; k < K; ++k) {
            const float *po = w + lstm_peep(l, q, k, 2);
            float so = q->sum_in_o[kb + k] + (first ? 0.f : q->sum_rec_o[kb + k]) + bo[k];
            for (size_t j = 0; j < cpb; ++j) so += q->c[cb + k * cpb + j] * po[j];
            q->sum_o[kb + k] = so;
            q->go[kb + k] = sigmoid_f(so);
            for (size_t j = 0; j < cpb; ++j) {
                size_t c = k * cpb + j;
                q->h[cb + c] = q->ca[cb + c] * q->go[kb + k];
                /* zoneout of the cell output (Forward_Pass__LSTM__Output__Zoneout, :1475-1478, :1520-1523) */
                if (zone && !q->zone_output[t * q->zone_stride + c]) q->h[cb + c] = first ? 0.f : q->h[cp + c];
            }
        }
    }
}

/* Forward_Pass__LSTM (NN/Neural_Network__Forward_Pass__OpenMP.cpp:1769-2340) of a normalised layer, one cell per block.
 * The eight sums of Gates_CIFO are normalised group by group and the gate functions take the normalised values
 * (Layer::Get__Array_Summations__*__Activation, NN/Neural_Network.cpp:4498-4613); the cell state is normalised before its
 * activation, while the recurrence, the peepholes and the forget path keep the raw cell state.  At the direction's first
 * step only groups 0, 3, 2 and 7 run (:1801-1829, :2014-2032, :2058-2074). */
static void fwd_lstm_step_norm(myea_oracle_net *n, size_t li, int dir, size_t t, size_t B)
{
    const myea_layer_desc *l = &n->d.layers[li];
    olayer *o = &n->L[li];
    olstm *q = &o->lstm[dir];
    size_t Bmax = n->d.batch_size, K = q->K, C = q->C, In = q->In;
    const float *x = layer_outputs(n, n->L[li].prev), *w = n->parameters;
    const float *bz = w + q->bias, *bi = bz + C, *bf = bi + K, *bo = bf + K;
    size_t tp = q->reverse ? t + 1 : t - 1;
    int first = q->reverse ? t == n->d.number_recurrent_depth - 1 : t == 0;
    int zone = l->type_dropout == MYEA_DROPOUT_ZONEOUT && n->state == MYEA_STATE_TRAINING;
    int renorm = l->type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
    long b;
#pragma omp parallel for schedule(static) num_threads(n->threads)
    for (b = 0; b < (long)B; ++b) {   /* Gates_CIFO */
        size_t kb = (size_t)b * K + Bmax * K * t, cp = (size_t)b * C + Bmax * C * tp;
        const float *xi = x + (size_t)b * In + Bmax * In * t;
        const float *hp = first ? NULL : q->h + cp;
        for (size_t k = 0; k < K; ++k) {
            float *in4[4] = {q->sum_in_z, q->sum_in_i, q->sum_in_f, q->sum_in_o}, *rec4[4] = {q->sum_rec_z, q->sum_rec_i, q->sum_rec_f, q->sum_rec_o};
            for (int g = 0; g < 4; ++g) {
                const float *wi = w + (g == 0 ? lstm_z_in(l, q, k, 0) : lstm_gate_in(l, q, k, g - 1));
                float v = 0.f;
                for (size_t a = 0; a < In; ++a) v += xi[a] * wi[a];
                in4[g][kb + k] = v;
                if (first) continue;
                const float *wr = w + (g == 0 ? lstm_z_rec(l, q, k, 0) : lstm_gate_rec(l, q, k, g - 1));
                v = 0.f;
                for (size_t a = 0; a < C; ++a) v += hp[a] * wr[a];
                rec4[g][kb + k] = v;
            }
        }
    }
    lstm_bn_forward(n, renorm, &q->nrm[0], t, B, q->sum_in_z);
    lstm_bn_forward(n, renorm, &q->nrm[3], t, B, q->sum_in_i);
    if (!first) {
        lstm_bn_forward(n, renorm, &q->nrm[5], t, B, q->sum_in_f);
        lstm_bn_forward(n, renorm, &q->nrm[1], t, B, q->sum_rec_z);
        lstm_bn_forward(n, renorm, &q->nrm[4], t, B, q->sum_rec_i);
        lstm_bn_forward(n, renorm, &q->nrm[6], t, B, q->sum_rec_f);
    }
    for (size_t bb = 0; bb < B; ++bb) {   /* Gates_CIF_AF_State on the normalised sums */
        size_t kb = bb * K + Bmax * K * t, cp = bb * C + Bmax * C * tp;
        for (size_t k = 0; k < K; ++k) {
            const float *pi = w + lstm_peep(l, q, k, 0), *pf = w + lstm_peep(l, q, k, 1);
            size_t c = kb + k;
            if (!first) {
                float si = q->nrm[3].normalizes[c] + q->nrm[4].normalizes[c] + bi[k];
                float sf = q->nrm[5].normalizes[c] + q->nrm[6].normalizes[c] + bf[k];
                si += q->c[cp + k] * pi[0]; sf += q->c[cp + k] * pf[0];
                q->sum_i[c] = si; q->sum_f[c] = sf;
                q->gi[c] = sigmoid_f(si); q->gf[c] = sigmoid_f(sf);
            } else {
                float si = q->nrm[3].normalizes[c] + bi[k];
                q->sum_i[c] = si;
                q->gi[c] = sigmoid_f(si);
            }
            float sz = first ? q->nrm[0].normalizes[c] + bz[k] : q->nrm[0].normalizes[c] + q->nrm[1].normalizes[c] + bz[k];
            q->sum_z[c] = sz;
            q->z[c] = tanh_f(sz);
            q->c[c] = first ? q->z[c] * q->gi[c] : q->z[c] * q->gi[c] + q->gf[c] * q->c[cp + k];
            if (zone && !q->zone_state[t * q->zone_stride + k]) q->c[c] = first ? 0.f : q->c[cp + k];
        }
    }
    lstm_bn_forward(n, renorm, &q->nrm[2], t, B, q->c);
    for (size_t bb = 0; bb < B; ++bb)   /* States_AF on the normalised cell state */
        for (size_t k = 0; k < C; ++k) { size_t c = bb * C + Bmax * C * t + k; q->ca[c] = tanh_f(q->nrm[2].normalizes[c]); }
    lstm_bn_forward(n, renorm, &q->nrm[7], t, B, q->sum_in_o);
    if (!first) lstm_bn_forward(n, renorm, &q->nrm[8], t, B, q->sum_rec_o);
    for (size_t bb = 0; bb < B; ++bb) {   /* Output */
        size_t kb = bb * K + Bmax * K * t, cp = bb * C + Bmax * C * tp;
        for (size_t k = 0; k < K; ++k) {
            const float *po = w + lstm_peep(l, q, k, 2);
            size_t c = kb + k;
            float so = q->nrm[7].normalizes[c] + (first ? 0.f : q->nrm[8].normalizes[c]) + bo[k];
            so += q->c[c] * po[0];
            q->sum_o[c] = so;
            q->go[c] = sigmoid_f(so);
            q->h[c] = q->ca[c] * q->go[c];
            if (zone && !q->zone_output[t * q->zone_stride + k]) q->h[c] = first ? 0.f : q->h[cp + k];
        }
    }
}

/* Backward_Pass__LSTM (NN/Neural_Network__Recurrent_Backward_Pass__OpenMP.cpp:1024-1120): delta to the layer below,
 * dst[t][b][:] += dz_c Wz_in[c][:] + di_k Wi_in[k][:] + df_k Wf_in[k][:] + do_k Wo_in[k][:] */
static void bwd_lstm_to_previous_dir(myea_oracle_net *n, size_t gi, int dir, size_t t, size_t B, float *dst)
{
    const myea_layer_desc *l = &n->d.layers[gi];
    olstm *q = &n->L[gi].lstm[dir];
    size_t Bmax = n->d.batch_size, K = q->K, C = q->C, cpb = q->cpb, In = q->In;
    const float *w = n->parameters;
    long b;
#pragma omp parallel for schedule(static) num_threads(n->threads)
    for (b = 0; b < (long)B; ++b) {
        size_t kb = (size_t)b * K + Bmax * K * t, cb = (size_t)b * C + Bmax * C * t;
        float *dx = dst + (size_t)b * In + Bmax * In * t;
        /* a normalised layer hands down the deltas of its sums from below, after their normalisation's backward pass
         * (Layer::Get__Array_Deltas__*__Input, NN/Neural_Network.cpp:4615-4717) */
        const float *dzs = q->norm ? q->dz_in : q->dz;
        for (size_t k = 0; k < K; ++k) {
            for (size_t j = 0; j < cpb; ++j) {
                float e = dzs[cb + k * cpb + j];
                const float *wr = w + lstm_z_in(l, q, k, j);
                for (size_t a = In; a--;) dx[a] += e * wr[a];
            }
            const float *d3[3] = {q->norm ? q->di_in : q->di, q->norm ? q->df_in : q->df, q->norm ? q->do_in : q->dgo};
            for (int g = 0; g < 3; ++g) {
                float e = d3[g][kb + k];
                const float *wr = w + lstm_gate_in(l, q, k, g);
                for (size_t a = In; a--;) dx[a] += e * wr[a];
            }
        }
    }
}

static void bwd_lstm_to_previous(myea_oracle_net *n, size_t gi, size_t t, size_t B, float *dst)
{
    bwd_lstm_to_previous_dir(n, gi, 0, t, B, dst);
    if (n->d.layers[gi].use_bidirectional) bwd_lstm_to_previous_dir(n, gi, 1, t, B, dst);
}

/* Recurrent__Backward_Pass__Gradient__LSTM (:440-862) for one time step, t descending:
 * Backward_Pass__LSTM_Derivative__Output (:1130-1273), __Cell_State_AF (:1275-1327), __Gates_CIF_AF_State (:1329-1604). */
static void bwd_lstm_step(myea_oracle_net *n, size_t li, int dir, size_t t, size_t B)
{
    const myea_layer_desc *l = &n->d.layers[li];
    olayer *o = &n->L[li];
    olstm *q = &o->lstm[dir];
    size_t Bmax = n->d.batch_size, T = n->d.number_recurrent_depth, K = q->K, C = q->C, cpb = q->cpb;
    const float *w = n->parameters;
    /* "next" / "previous" in the direction's own processing order */
    size_t tn = q->reverse ? t - 1 : t + 1, tp = q->reverse ? t + 1 : t - 1;
    int last = q->reverse ? t == 0 : t == T - 1, first = q->reverse ? t == T - 1 : t == 0;
    long b;
#pragma omp parallel for schedule(static) num_threads(n->threads)
    for (b = 0; b < (long)B; ++b) {
        size_t kb = (size_t)b * K + Bmax * K * t, cb = (size_t)b * C + Bmax * C * t;
        size_t kn = (size_t)b * K + Bmax * K * tn, cn = (size_t)b * C + Bmax * C * tn, cp = (size_t)b * C + Bmax * C * tp;
        float *dh = q->dh + cb;
        if (!last) { /* recurrent delta from t + 1: of the recurrent sums when the layer is normalised (Get__Array_Deltas__*__Recurrent) */
            const float *rz = q->norm ? q->dz_rec : q->dz, *ri = q->norm ? q->di_rec : q->di, *rf = q->norm ? q->df_rec : q->df, *ro = q->norm ? q->do_rec : q->dgo;
            for (size_t c = 0; c < C; ++c) {
                float e = rz[cn + c];
                const float *wr = w + lstm_z_rec(l, q, c / cpb, c % cpb);
                for (size_t a = 0; a < C; ++a) dh[a] += e * wr[a];
            }
            for (size_t k = 0; k < K; ++k) {
                float ei = ri[kn + k], ef = rf[kn + k], eo = ro[kn + k];
                const float *wi = w + lstm_gate_rec(l, q, k, 0), *wf = w + lstm_gate_rec(l, q, k, 1), *wo = w + lstm_gate_rec(l, q, k, 2);
                for (size_t a = C; a--;) { float e = ei * wi[a]; e += ef * wf[a]; e += eo * wo[a]; dh[a] += e; }
            }
        }
        for (size_t k = 0; k < K; ++k) { /* output gate */
            float e = 0.f;
            for (size_t j = 0; j < cpb; ++j) e += dh[k * cpb + j] * q->ca[cb + k * cpb + j];
            float a = q->go[kb + k];
            q->dgo[kb + k] = (1.f * a * (1.f - a)) * e;
        }
        for (size_t k = 0; k < K; ++k) /* cell state through tanh, on the stored activation */
            for (size_t j = 0; j < cpb; ++j) {
                size_t c = k * cpb + j;
                q->dc[cb + c] = dh[c] * q->go[kb + k] * (1.f * (1.f - q->ca[cb + c] * q->ca[cb + c]));
            }
        if (first && last) continue; /* T == 1: no branch of Gates_CIF_AF_State matches */
        for (size_t k = 0; k < K; ++k) {
            const float *pi = w + lstm_peep(l, q, k, 0), *pf = w + lstm_peep(l, q, k, 1), *po = w + lstm_peep(l, q, k, 2);
            float gi_ = q->gi[kb + k], ddo = q->dgo[kb + k];
            for (size_t j = 0; j < cpb; ++j) {
                size_t c = k * cpb + j;
                float e = q->dc[cb + c];
                e += po[j] * ddo;
                if (!last) {
                    e += pi[j] * q->di[kn + k];
                    e += pf[j] * q->df[kn + k];
                    e += q->dc[cn + c] * q->gf[kn + k];
                }
                q->dc[cb + c] = e;
                q->dz[cb + c] = e * gi_ * (1.f * (1.f - q->z[cb + c] * q->z[cb + c]));
            }
            float ei = 0.f, ef = 0.f;
            for (size_t j = 0; j < cpb; ++j) {
                size_t c = k * cpb + j;
                ei += q->dc[cb + c] * q->z[cb + c];
                if (!first) ef += q->dc[cb + c] * q->c[cp + c];
            }
            q->di[kb + k] = ei * (1.f * gi_ * (1.f - gi_));
            if (!first) { float f = q->gf[kb + k]; q->df[kb + k] = ef * (1.f * f * (1.f - f)); } /* df[0] is never written */
        }
    }
}

/* The same time step of a normalised layer (one cell per block), NN/Neural_Network__Recurrent_Backward_Pass__OpenMP.cpp:476-862:
 * Output -> [output gate's delta copied to its two sums' deltas, each through its normalisation] -> Cell_State_AF ->
 * [cell state's delta through its normalisation, in place] -> Gates_CIF_AF_State -> [block input, input gate and forget
 * gate deltas copied to their sums' deltas, each through its normalisation].  The recurrent sums have no delta at the
 * direction's first step, and there the forget gate's sum from below is copied but not passed through (:650-664, :706-741). */
static void bwd_lstm_step_norm(myea_oracle_net *n, size_t li, int dir, size_t t, size_t B)
{
    const myea_layer_desc *l = &n->d.layers[li];
    olayer *o = &n->L[li];
    olstm *q = &o->lstm[dir];
    size_t Bmax = n->d.batch_size, T = n->d.number_recurrent_depth, K = q->K, C = q->C;
    const float *w = n->parameters;
    size_t tn = q->reverse ? t - 1 : t + 1, tp = q->reverse ? t + 1 : t - 1;
    int last = q->reverse ? t == 0 : t == T - 1, first = q->reverse ? t == T - 1 : t == 0;
    int renorm = l->type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
    size_t row0 = Bmax * K * t, bytes = B * K * sizeof(float);
    long b;
#pragma omp parallel for schedule(static) num_threads(n->threads)
    for (b = 0; b < (long)B; ++b) {
        size_t kb = (size_t)b * K + row0, kn = (size_t)b * K + Bmax * K * tn;
        float *dh = q->dh + kb;
        if (!last) {
            for (size_t c = 0; c < C; ++c) {
                float e = q->dz_rec[kn + c];
                const float *wr = w + lstm_z_rec(l, q, c, 0);
                for (size_t a = 0; a < C; ++a) dh[a] += e * wr[a];
            }
            for (size_t k = 0; k < K; ++k) {
                float ei = q->di_rec[kn + k], ef = q->df_rec[kn + k], eo = q->do_rec[kn + k];
                const float *wi = w + lstm_gate_rec(l, q, k, 0), *wf = w + lstm_gate_rec(l, q, k, 1), *wo = w + lstm_gate_rec(l, q, k, 2);
                for (size_t a = C; a--;) { float e = ei * wi[a]; e += ef * wf[a]; e += eo * wo[a]; dh[a] += e; }
            }
        }
        for (size_t k = 0; k < K; ++k) {
            float a = q->go[kb + k];
            q->dgo[kb + k] = (1.f * a * (1.f - a)) * (dh[k] * q->ca[kb + k]);
        }
    }
    memcpy(q->do_in + row0, q->dgo + row0, bytes);
    lstm_bn_backward(n, renorm, &q->nrm[7], t, B, q->sum_in_o, q->do_in);
    if (!first) {
        memcpy(q->do_rec + row0, q->dgo + row0, bytes);
        lstm_bn_backward(n, renorm, &q->nrm[8], t, B, q->sum_rec_o, q->do_rec);
    }
    for (size_t bb = 0; bb < B; ++bb)
        for (size_t k = 0; k < K; ++k) {
            size_t c = bb * K + row0 + k;
            q->dc[c] = q->dh[c] * q->go[c] * (1.f * (1.f - q->ca[c] * q->ca[c]));
        }
    lstm_bn_backward(n, renorm, &q->nrm[2], t, B, q->c, q->dc);
    if (!(first && last))
        for (size_t bb = 0; bb < B; ++bb) {
            size_t kb = bb * K + row0, kn = bb * K + Bmax * K * tn, cp = bb * C + Bmax * C * tp;
            for (size_t k = 0; k < K; ++k) {
                const float *pi = w + lstm_peep(l, q, k, 0), *pf = w + lstm_peep(l, q, k, 1), *po = w + lstm_peep(l, q, k, 2);
                float gi_ = q->gi[kb + k];
                float e = q->dc[kb + k];
                e += po[0] * q->dgo[kb + k];
                if (!last) {
                    e += pi[0] * q->di[kn + k];
                    e += pf[0] * q->df[kn + k];
                    e += q->dc[kn + k] * q->gf[kn + k];
                }
                q->dc[kb + k] = e;
                q->dz[kb + k] = e * gi_ * (1.f * (1.f - q->z[kb + k] * q->z[kb + k]));
                q->di[kb + k] = (e * q->z[kb + k]) * (1.f * gi_ * (1.f - gi_));
                if (!first) { float f = q->gf[kb + k]; q->df[kb + k] = (e * q->c[cp + k]) * (1.f * f * (1.f - f)); }
            }
        }
    memcpy(q->dz_in + row0, q->dz + row0, bytes);
    memcpy(q->di_in + row0, q->di + row0, bytes);
    memcpy(q->df_in + row0, q->df + row0, bytes);
    if (!first) {
        memcpy(q->dz_rec + row0, q->dz + row0, bytes);
        memcpy(q->di_rec + row0, q->di + row0, bytes);
        memcpy(q->df_rec + row0, q->df + row0, bytes);
    }
    lstm_bn_backward(n, renorm, &q->nrm[0], t, B, q->sum_in_z, q->dz_in);
    lstm_bn_backward(n, renorm, &q->nrm[3], t, B, q->sum_in_i, q->di_in);
    if (!first) {
        lstm_bn_backward(n, renorm, &q->nrm[5], t, B, q->sum_in_f, q->df_in);
        lstm_bn_backward(n, renorm, &q->nrm[1], t, B, q->sum_rec_z, q->dz_rec);
        lstm_bn_backward(n, renorm, &q->nrm[4], t, B, q->sum_rec_i, q->di_rec);
        lstm_bn_backward(n, renorm, &q->nrm[6], t, B, q->sum_rec_f, q->df_rec);
    }
}

/* Recurrent__Update_Derivative_Weight__LSTM (NN/Neural_Network__Recurrent_Update_Derivative_Weight__OpenMP.cpp:492-728)
 * and __LSTM__Bias (:730-776). */
static void dw_lstm_dir(myea_oracle_net *n, size_t li, int dir, size_t B)
{
    const myea_layer_desc *l = &n->d.layers[li];
    olayer *o = &n->L[li];
    olstm *q = &o->lstm[dir];
    size_t Bmax = n->d.batch_size, T = n->d.number_recurrent_depth, K = q->K, C = q->C, cpb = q->cpb, In = q->In;
    const float *x = layer_outputs(n, n->L[li].prev);
    float *g = n->gradient;
    long kk;
    /* a normalised layer: the weights from below take the deltas of the sums from below, the recurrent weights those of the
     * recurrent sums, each after its normalisation's backward pass; the input and forget peepholes take the RECURRENT sums'
     * deltas of the next step and the output peephole the delta of the output gate's sum FROM BELOW (the variables the
     * reference's loop happens to hold at that point, :601-617, :688-696); the biases take the gates' own deltas (:730-776) */
    const float *z_in = q->norm ? q->dz_in : q->dz, *z_rec = q->norm ? q->dz_rec : q->dz;
    const float *i_in = q->norm ? q->di_in : q->di, *i_rec = q->norm ? q->di_rec : q->di;
    const float *f_in = q->norm ? q->df_in : q->df, *f_rec = q->norm ? q->df_rec : q->df;
    const float *o_in = q->norm ? q->do_in : q->dgo, *o_rec = q->norm ? q->do_rec : q->dgo;
    /* parallel over blocks: every parameter belongs to one block, so the per-parameter summation order (b, then t)
     * is the serial one */
#pragma omp parallel for schedule(static) num_threads(n->threads)
    for (kk = 0; kk < (long)K; ++kk) {
        size_t k = (size_t)kk;
        for (size_t b = 0; b < B; ++b)
            for (size_t t = 0; t < T; ++t) {
                int last = q->reverse ? t == 0 : t == T - 1;
                size_t tn = q->reverse ? t - 1 : t + 1;
                size_t kb = b * K + Bmax * K * t, cb = b * C + Bmax * C * t, kn = b * K + Bmax * K * tn, cn = b * C + Bmax * C * tn;
                const float *xi = x + b * In + Bmax * In * t, *h = q->h + cb;
                for (size_t j = 0; j < cpb; ++j) {
                    size_t c = k * cpb + j;
                    float e = z_in[cb + c];
                    float *gw = g + lstm_z_in(l, q, k, j);
                    for (size_t a = 0; a < In; ++a) gw[a] += e * xi[a];
                    if (!last) {
                        e = z_rec[cn + c];
                        gw = g + lstm_z_rec(l, q, k, j);
                        for (size_t a = 0; a < C; ++a) gw[a] += e * h[a];
                    }
                }
                float ei = i_in[kb + k], ef = f_in[kb + k], eo = o_in[kb + k];
                float *gi_ = g + lstm_gate_in(l, q, k, 0), *gf_ = g + lstm_gate_in(l, q, k, 1), *go_ = g + lstm_gate_in(l, q, k, 2);
                for (size_t a = 0; a < In; ++a) { gi_[a] += ei * xi[a]; gf_[a] += ef * xi[a]; go_[a] += eo * xi[a]; }
                float *pi = g + lstm_peep(l, q, k, 0), *pf = g + lstm_peep(l, q, k, 1), *po = g + lstm_peep(l, q, k, 2);
                if (!last) {
                    ei = i_rec[kn + k]; ef = f_rec[kn + k];
                    for (size_t j = 0; j < cpb; ++j) { float cs = q->c[cb + k * cpb + j]; pi[j] += ei * cs; pf[j] += ef * cs; po[j] += eo * cs; }
                    eo = o_rec[kn + k];
                    gi_ = g + lstm_gate_rec(l, q, k, 0); gf_ = g + lstm_gate_rec(l, q, k, 1); go_ = g + lstm_gate_rec(l, q, k, 2);
                    for (size_t a = 0; a < C; ++a) { gi_[a] += ei * h[a]; gf_[a] += ef * h[a]; go_[a] += eo * h[a]; }
                } else {
                    for (size_t j = 0; j < cpb; ++j) po[j] += eo * q->c[cb + k * cpb + j];
                }
            }
    }
    float *bz = g + q->bias, *bi = bz + C, *bf = bi + K, *bo = bf + K;
    for (size_t b = 0; b < B; ++b)
        for (size_t t = 0; t < T; ++t) {
            size_t kb = b * K + Bmax * K * t, cb = b * C + Bmax * C * t;
            for (size_t c = 0; c < C; ++c) bz[c] += q->dz[cb + c];
            for (size_t k = 0; k < K; ++k) { bi[k] += q->di[kb + k]; bf[k] += q->df[kb + k]; bo[k] += q->dgo[kb + k]; }
        }
}

static void dw_lstm(myea_oracle_net *n, size_t li, size_t B)
{
    dw_lstm_dir(n, li, 0, B);
    if (n->d.layers[li].use_bidirectional) dw_lstm_dir(n, li, 1, B);
}

/* A layer with two directions (contract of this library; the reference's own two-direction path overlays the
 * directions' buffers and cannot be followed): each direction is the one-direction recurrence above over its own blocks,
 * the second one walking time backwards; the layer's output is the SUM of the two cell outputs (the layer keeps the
 * width of one direction, NN/Neural_Network__Compile.cpp:79) and both directions receive the same delta from above
 * (NN/Neural_Network__Recurrent_Backward_Pass__OpenMP.cpp:144-156). */
static void fwd_lstm_layer(myea_oracle_net *n, size_t li, size_t B)
{
    olayer *o = &n->L[li];
    size_t T = n->d.number_recurrent_depth, dirs = n->d.layers[li].use_bidirectional ? 2 : 1;
    for (size_t dir = 0; dir < dirs; ++dir)
        for (size_t s = 0; s < T; ++s) (o->lstm[dir].norm ? fwd_lstm_step_norm : fwd_lstm_step)(n, li, (int)dir, dir ? T - 1 - s : s, B);
    if (dirs == 2) {
        size_t cnt = T * n->d.batch_size * o->H;
        for (size_t i = 0; i < cnt; ++i) o->values[i] = o->lstm[0].h[i] + o->lstm[1].h[i];
    }
}

static void bwd_lstm_layer(myea_oracle_net *n, size_t li, size_t B)
{
    olayer *o = &n->L[li];
    size_t T = n->d.number_recurrent_depth, dirs = n->d.layers[li].use_bidirectional ? 2 : 1;
    for (size_t dir = 0; dir < dirs; ++dir) {
        if (dirs == 2) memcpy(o->lstm[dir].dh, o->af_errors, T * n->d.batch_size * o->H * sizeof(float));
        for (size_t s = T; s-- > 0;) (o->lstm[dir].norm ? bwd_lstm_step_norm : bwd_lstm_step)(n, li, (int)dir, dir ? T - 1 - s : s, B);
    }
}

/* FF__Forward_Pass_Batch: NN/Neural_Network__Forward_Pass__OpenMP.cpp:24-120;
 * RNN__Forward_Pass_Batch: NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:24-130 (layer-major,
 * every layer loops over t); FF/RNN__Assign_Inputs: NN/Neural_Network__Assign_Inputs.cpp:20-204
 * (example rows are [T][In]; scattered into [T][Bmax][In]; input-layer dropout applied in place). */
/* Forward_Pass__Average_Pooling / __Max_Pooling (NN/Neural_Network__Forward_Pass__Loop.cpp:4537-4583, 5070-5135): windows over the
 * feature axis of one example; positions are counted in the padded coordinate p = output * stride + k * dilation, the input
 * sits at [padding, padding + In).  Average: padding contributes 0 and the divisor is always the kernel size.  Max: a padded
 * position stands for the value 0; the index kept for the backward pass is the padded coordinate of the first maximum. */
static void fwd_pooling(myea_oracle_net *n, size_t li, size_t t, size_t B)
{
    const myea_layer_desc *l = &n->d.layers[li];
    olayer *o = &n->L[li];
    size_t Bmax = n->d.batch_size, In = o->In, H = o->H;
    size_t kernel = l->pooling_values[0], stride = l->pooling_values[1], padding = l->pooling_values[2], dilation = l->pooling_values[3];
    const float *x = layer_outputs(n, o->prev) + Bmax * In * t;
    float *y = o->values + Bmax * H * t;
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) {
            if (l->type_layer == MYEA_LAYER_AVERAGE_POOLING) {
                float s = 0.f;
                for (size_t k = 0; k < kernel; ++k) {
                    size_t p = j * stride + k * dilation;
                    if (p < padding || p >= In + padding) continue;
                    s += x[b * In + p - padding];
                }
                y[b * H + j] = s * (1.f / (float)kernel);
            } else {
                size_t at = 0; float mx = -FLT_MAX;
                for (size_t k = 0; k < kernel; ++k) {
                    size_t p = j * stride + k * dilation;
                    if (p < padding || p >= In + padding) { if (mx < 0.f) { at = p; mx = 0.f; } }
                    else if (mx < x[b * In + p - padding]) { at = p; mx = x[b * In + p - padding]; }
                }
                o->pool_index[Bmax * H * t + b * H + j] = (uint32_t)at;
                y[b * H + j] = mx;
            }
        }
}

/* Backward_Pass__Average_Pooling / __Max_Pooling (NN/Neural_Network__Backward_Pass__Loop.cpp:1004-1049, 1139-1181): the pooling layer
 * ci hands its errors down to `dst` (the previous layer's derivative outputs, In wide), added in place */
static void bwd_pooling_to_previous(myea_oracle_net *n, size_t ci, size_t t, size_t B, float *dst)
{
    const myea_layer_desc *l = &n->d.layers[ci];
    olayer *o = &n->L[ci];
    size_t Bmax = n->d.batch_size, In = o->In, H = o->H;
    size_t kernel = l->pooling_values[0], stride = l->pooling_values[1], padding = l->pooling_values[2], dilation = l->pooling_values[3];
    const float *dy = o->af_errors + Bmax * H * t;
    float *dx = dst + Bmax * In * t;
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) {
            if (l->type_layer == MYEA_LAYER_AVERAGE_POOLING) {
                float e = dy[b * H + j] * (1.f / (float)kernel);
                for (size_t k = 0; k < kernel; ++k) {
                    size_t p = j * stride + k * dilation;
                    if (p < padding || p >= In + padding) continue;
                    dx[b * In + p - padding] += e;
                }
            } else {
                size_t p = o->pool_index[Bmax * H * t + b * H + j];
                if (p < padding || p >= In + padding) continue;
                dx[b * In + p - padding] += dy[b * H + j];
            }
        }
}

int myea_oracle_forward_pass(myea_oracle_net *n, size_t B, const float *inputs)
{
    if (!n || !inputs) return MYEA_E_INVALID;
    size_t Bmax = n->d.batch_size, T = n->d.number_recurrent_depth, In = n->L[0].H;
    if (B > Bmax) return MYEA_E_BATCH;
    for (size_t b = 0; b < B; ++b)
        for (size_t t = 0; t < T; ++t)
            memcpy(n->L[0].values + Bmax * In * t + b * In, inputs + b * T * In + t * In, In * sizeof(float));
    for (size_t t = 0; t < T; ++t) fwd_dropout(n, &n->d.layers[0], t, B, In, n->L[0].values);
    for (size_t li = 1; li < n->d.n_layers; ++li) {
        const myea_layer_desc *l = &n->d.layers[li];
        if (is_dense(l)) {
            for (size_t t = 0; t < T; ++t) fwd_fc_layer(n, li, t, B);
        } else if (l->type_layer == MYEA_LAYER_LSTM) {
            fwd_lstm_layer(n, li, B);
        } else if (l->type_layer == MYEA_LAYER_RESIDUAL) {
            fwd_residual_members(n, li, B);
            for (size_t t = 0; t < T; ++t) fwd_residual_block(n, li, t, B);
            li += l->block_depth; /* the iterator is left on the block's last member, :3884-3885 */
        } else if (is_pooling(l)) {
            for (size_t t = 0; t < T; ++t) fwd_pooling(n, li, t, B);
        } else return MYEA_E_UNSUPPORTED;
    }
    return MYEA_OK;
}

/* ------------------------------------------------------------------------------------------- */
/* Compute__Error */

/* Update_Error: NN/Neural_Network__Compute__Error__Loop.cpp:20-77 */
static void update_error(myea_oracle_net *n, float observed, float desired, float error)
{
    float e;
    switch (n->h.type_loss_function) {
    case MYEA_LOSS_ME:
    case MYEA_LOSS_L1: e = error; break;
    case MYEA_LOSS_MAE: e = fabsf(error); break;
    case MYEA_LOSS_L2:
    case MYEA_LOSS_MSE:
    case MYEA_LOSS_RMSE: e = error * error; break;
    case MYEA_LOSS_MAPE:
        e = observed != 0.f ? observed : (observed > 1e-6f ? observed : 1e-6f);
        e = fabsf(error / e);
        break;
    case MYEA_LOSS_SMAPE: e = fabsf(error) / (fabsf(desired) + fabsf(observed)); break;
    case MYEA_LOSS_CROSS_ENTROPY: {
        size_t n_out = n->L[n->d.n_layers - 1].H;
        e = observed != 0.f ? observed : (observed > 1e-6f ? observed : 1e-6f);
        if (n_out == 1) e = -(desired * logf(e) + (1.f - desired) * logf(1.f - e));
        else e = -(desired * logf(e));
        break;
    }
    case MYEA_LOSS_BIT:
        if (fabsf(error) >= n->h.bit_fail_limit) ++n->loss.number_bit_fail;
        return;
    default: return;
    }
    n->loss.loss_values += e;
    ++n->loss.number_loss;
}

static float sign_f(float v) { return v > 0.f ? 1.f : (v < 0.f ? -1.f : 0.f); }

/* FF__Compute__Error: NN/Neural_Network__Compute__Error__OpenMP.cpp:22-141.
 * RNN__Compute__Error: NN/Neural_Network__Recurrent_Compute__Error__OpenMP.cpp:22-159 — same per
 * t >= number_time_delays; its per-unit loop does not advance the pre-activation pointer (:97-99),
 * so every unit of an example sees the first unit's pre-activation.  Only activations whose derivative
 * ignores the pre-activation (linear, tanh, sigmoid, softmax) are unaffected; this restatement
 * reproduces the quirk.
 * delta = Activation_Function_Derive(type, pre, steepness, y) * (y - desired); no 1/B, no factor 2. */
static int compute_error_or_loss(myea_oracle_net *n, size_t B, const float *desired, int write_delta)
{
    if (!n || !desired) return MYEA_E_INVALID;
    size_t Bmax = n->d.batch_size, T = n->d.number_recurrent_depth;
    if (B > Bmax) return MYEA_E_BATCH;
    size_t lo = n->d.n_layers - 1;
    const myea_layer_desc *l = &n->d.layers[lo];
    olayer *o = &n->L[lo];
    size_t H = o->H;
    const float *pre_af = (layer_uses_norm(l) && l->use_layer_normalization_before_activation) ? o->normalizes : o->summations;
    int rnn = T > 1;
    for (size_t t = rnn ? n->h.number_time_delays : 0; t < T; ++t) {
        size_t off = Bmax * H * t;
        for (size_t b = 0; b < B; ++b) {
            const float *y = o->values + off + b * H;
            const float *d = desired + b * T * H + t * H;
            const float *pre = pre_af + off + b * H;
            float *err = o->af_errors + off + b * H;
            if (n->h.type_accuracy_function == MYEA_ACCURACY_CROSS_ENTROPY) {
                size_t want = 0, got = 0;
                for (want = 0; want < H; ++want) if (d[want] == 1.f) break;
                float mx = -FLT_MAX;
                for (size_t j = 0; j < H; ++j) if (y[j] >= mx) { got = j; mx = y[j]; }
                n->loss.accuracy_value += (double)(want == got);
            }
            for (size_t j = 0; j < H; ++j) {
                float diff = y[j] - d[j];
                update_error(n, y[j], d[j], diff);
                switch (n->h.type_accuracy_function) {
                case MYEA_ACCURACY_DISTANCE: if (fabsf(diff) <= n->h.accuracy_variance) n->loss.accuracy_value += 1.0; break;
                case MYEA_ACCURACY_DIRECTIONAL:
                    /* RNN: direction of change against the previous target (NN/Neural_Network__Recurrent_Compute__Error__OpenMP.cpp:115-120) */
                    if (!rnn || t == 0 || sign_f(d[j] - (d - H)[j]) == sign_f(y[j] - (d - H)[j])) n->loss.accuracy_value += 1.0;
                    break;
                case MYEA_ACCURACY_SIGN:
                    if (sign_f(d[j]) == sign_f(y[j]) || (sign_f(d[j]) == 0.f && y[j] >= -FLT_EPSILON && y[j] <= FLT_EPSILON)) n->loss.accuracy_value += 1.0;
                    break;
                case MYEA_ACCURACY_R: /* running sums; the means are taken by the caller (NN/Neural_Network__Compute__Error__Loop.cpp:173-176) */
                    n->loss.accuracy_value += d[j];
                    n->loss.accuracy_r[0] += y[j];
                    break;
                default: break;
                }
                if (!write_delta) continue;
                float q = rnn ? pre[0] : pre[j];
                err[j] = myea_oracle_activation_derive(o->unit_af ? o->unit_af[j] : l->type_activation_function, q, o->unit_steep ? o->unit_steep[j] : l->activation_steepness, y[j]) * diff;
            }
        }
    }
    /* MEMCPY AF errors -> neuron errors over batch_size * T * H (:136-139) */
    if (write_delta) memcpy(o->neuron_errors, o->af_errors, T * Bmax * H * sizeof(float));
    return MYEA_OK;
}

int myea_oracle_compute_error(myea_oracle_net *n, size_t B, const float *desired) { return compute_error_or_loss(n, B, desired, 1); }

/* FF__Compute__Loss / RNN__Compute__Loss (NN/Neural_Network__Compute__Loss__Loop.cpp:39-140,
 * NN/Neural_Network__Recurrent_Compute__Loss__Loop.cpp:20-140): the same accumulation, no delta */
int myea_oracle_compute_loss(myea_oracle_net *n, size_t B, const float *desired) { return compute_error_or_loss(n, B, desired, 0); }

/* FF / RNN__Compute__Accuracy__R (NN/Neural_Network__Compute__R__Loop.cpp:38-90, NN/Neural_Network__Recurrent_Compute__R__Loop.cpp:20-75) */
int myea_oracle_compute_accuracy_r(myea_oracle_net *n, size_t B, const float *desired, float desired_mean, float predicted_mean)
{
    if (!n || !desired) return MYEA_E_INVALID;
    size_t Bmax = n->d.batch_size, T = n->d.number_recurrent_depth;
    if (B > Bmax) return MYEA_E_BATCH;
    olayer *o = &n->L[n->d.n_layers - 1];
    size_t H = o->H;
    for (size_t b = 0; b < B; ++b)
        for (size_t t = T > 1 ? n->h.number_time_delays : 0; t < T; ++t) {
            const float *y = o->values + Bmax * H * t + b * H, *d = desired + b * T * H + t * H;
            for (size_t j = 0; j < H; ++j) {
                float dd = d[j] - desired_mean, dy = y[j] - predicted_mean;
                n->loss.accuracy_r[1] += dd * dy;
                n->loss.accuracy_r[2] += dd * dd;
                n->loss.accuracy_r[3] += dy * dy;
            }
        }
    return MYEA_OK;
}

/* ------------------------------------------------------------------------------------------- */
/* backward pieces */

/* Backward_Pass__FC (7-arg): NN/Neural_Network__Backward_Pass__OpenMP.cpp:1044-1082.
 * dst[b][i] += sum_o delta[b][o] * W[o][i]; dst is pre-zeroed by the driver. */
static void bwd_fc(myea_oracle_net *n, size_t t, size_t B, size_t Out, size_t In, const float *delta, const float *w, float *dst)
{
    size_t Bmax = n->d.batch_size;
    const float *dt = delta + Bmax * Out * t;
    float *xt = dst + Bmax * In * t;
    long b;
#pragma omp parallel for schedule(static) num_threads(n->threads)
    for (b = 0; b < (long)B; ++b) {
        const float *di = dt + (size_t)b * Out;
        float *xo = xt + (size_t)b * In;
        for (size_t o = 0; o < Out; ++o) {
            float e = di[o];
            const float *wr = w + o * In;
            for (size_t i = 0; i < In; ++i) xo[i] += e * wr[i];
        }
    }
}

/* Backward_Pass__FC__DF: :1225-1263 */
static void bwd_df(myea_oracle_net *n, size_t t, size_t B, size_t H, uint32_t type, float steep, const uint32_t *unit_type, const float *unit_steep,
                   const float *pre, const float *val, const float *dy, float *dx)
{
    size_t off = n->d.batch_size * H * t;
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) {
            size_t k = off + b * H + j;
            dx[k] = dy[k] * myea_oracle_activation_derive(unit_type ? unit_type[j] : type, pre[k], unit_steep ? unit_steep[j] : steep, val[k]);
        }
}

/* Backward_Pass__FC__DF_Ind_RNN (NN/Neural_Network__Backward_Pass__Loop.cpp:1296-1390): errors = dY * AF'(t);
 * dAF(t) = errors + u * AF'(t) * dAF(t+1), without the second term at the last time step.  dAF is what the layer hands on
 * (to its normalisation, its neuron errors and the self-weight gradient). */
static void bwd_df_ind_rnn(myea_oracle_net *n, size_t t, size_t B, size_t H, const float *u, uint32_t type, float steep, const uint32_t *unit_type,
                           const float *unit_steep, const float *pre, const float *val, const float *dy, float *dafs, float *errors)
{
    size_t Bmax = n->d.batch_size, off = Bmax * H * t, next = Bmax * H * (t + 1);
    int last = t + 1 == n->d.number_recurrent_depth;
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) {
            size_t k = off + b * H + j;
            float daf = myea_oracle_activation_derive(unit_type ? unit_type[j] : type, pre[k], unit_steep ? unit_steep[j] : steep, val[k]);
            errors[k] = dy[k] * daf;
            dafs[k] = last ? errors[k] : errors[k] + u[j] * daf * dafs[next + b * H + j];
        }
}

/* Backward_Pass__Batch_Normalization: :1346-1467; Backward_Pass__Batch_Renormalization: :1586-1709.
 * dScale / dShift accumulate into the gradient vector at the scale / shift slots. */
static void bwd_bn(myea_oracle_net *n, int renorm, size_t li, size_t t, size_t B, size_t H,
                   const float *x, const float *dy, float *dx)
{
    olayer *o = &n->L[li];
    size_t Bmax = n->d.batch_size, off = Bmax * H * t;
    const float *mean = o->means + t * H, *var = o->variances + t * H, *rc = o->r_corrections + t * H;
    const float *scale = scale_ptr(n, n->parameters, li);
    float *dscale = scale_ptr(n, n->gradient, li), *dshift = shift_ptr(n, n->gradient, li);
    float *dmean = o->derivatives_means + t * H, *dvar = o->derivatives_variances + t * H;
    float bscale = 1.f / (float)B;
    for (size_t j = 0; j < H; ++j) { dmean[j] = 0.f; dvar[j] = 0.f; } /* MEMSET at the start of the pass, :54-68 */
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) {
            size_t k = off + b * H + j;
            float e = dy[k], vb = var[j], r = renorm ? rc[j] : 1.f;
            dscale[j] += e * o->hats[k];
            dshift[j] += e;
            e *= scale[j];
            dmean[j] += e * (-r / vb);
            dvar[j] += e * (x[k] - mean[j]) * (-r / (vb * vb));
            dx[k] = e;
        }
    for (size_t b = 0; b < B; ++b)
        for (size_t j = 0; j < H; ++j) {
            size_t k = off + b * H + j;
            float e = dx[k], vb = var[j], r = renorm ? rc[j] : 1.f;
            e *= r / vb;
            e += dvar[j] * ((x[k] - mean[j]) / ((float)B * vb));
            e += dmean[j] * bscale;
            dx[k] = e;
        }
}

/* Backward_Pass__Gradient__FC: :544-709 — [BN after] -> act' -> [BN before] -> copy to neuron errors */
static void bwd_gradient_fc(myea_oracle_net *n, size_t li, size_t t, size_t B)
{
    const myea_layer_desc *l = &n->d.layers[li];
    olayer *o = &n->L[li];
    size_t H = o->H, Bmax = n->d.batch_size;
    int renorm = l->type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
    int before = l->use_layer_normalization_before_activation;
    const float *cur = layer_derivative_outputs(n, li);
    if (layer_uses_norm(l) && !before) {
        bwd_bn(n, renorm, li, t, B, H, o->values /* pre_normalization */, cur, o->norm_errors);
        cur = o->norm_errors;
    }
    const float *pre_af = (layer_uses_norm(l) && before) ? o->normalizes : o->summations;
    if (is_ind_rnn(l)) {
        bwd_df_ind_rnn(n, t, B, H, n->parameters + l->first_connection_index + H * o->In, l->type_activation_function, l->activation_steepness,
                       o->unit_af, o->unit_steep, o->pre_afs, o->values, cur, o->dafs, o->af_errors);
        cur = o->dafs;
    } else {
        bwd_df(n, t, B, H, l->type_activation_function, l->activation_steepness, o->unit_af, o->unit_steep, pre_af, o->values, cur, o->af_errors);
        cur = o->af_errors;
    }
    if (layer_uses_norm(l) && before) {
        bwd_bn(n, renorm, li, t, B, H, o->summations /* pre_normalization */, cur, o->norm_errors);
        cur = o->norm_errors;
    }
    memcpy(o->neuron_errors + Bmax * H * t, cur + Bmax * H * t, Bmax * H * sizeof(float));
}

/* Backward_Pass__Residual (7-arg): NN/Neural_Network__Backward_Pass__OpenMP.cpp:1155-1215.  Shortcut gradient:
 * dst (width D) += the residual layer's errors (width R >= D), cropped at `pad` when R > D. */
static void bwd_residual_shortcut(myea_oracle_net *n, size_t t, size_t B, size_t R, size_t D, size_t pad, const float *err, float *dst)
{
    err += t * n->d.batch_size * R;
    dst += t * n->d.batch_size * D;
    for (size_t b = 0; b < B; ++b) {
        const float *e = err + b * R;
        float *d = dst + b * D;
        if (R == D) for (size_t j = 0; j < R; ++j) d[j] += e[j];
        else if (R > D) for (size_t j = 0; j < D; ++j) d[j] += e[j + pad];
        else for (size_t j = 0; j < R; ++j) d[j + pad] += e[j];
    }
}

/* Backward_Pass__Residual__FC: :454-534 - what a block member hands to its producer.  A member that is not the block's
 * first layer has already reduced its delta to its input side (Backward_Pass__Gradient__Residual__FC), so the producer
 * receives a COPY of those errors; the block's first layer ADDS (its producer also receives the shortcut): its
 * normalisation errors when it is normalised, delta * W otherwise. */
static void bwd_residual_fc_to_previous(myea_oracle_net *n, size_t gi, size_t t, size_t B, float *dst)
{
    const myea_layer_desc *g = &n->d.layers[gi];
    olayer *q = &n->L[gi];
    size_t Bmax = n->d.batch_size, D = q->In, at = t * Bmax * D;
    if (q->group == 2) memcpy(dst + at, (layer_uses_norm(g) ? q->norm_errors : (is_ind_rnn(g) ? q->dafs : q->af_errors)) + at, Bmax * D * sizeof(float));
    else if (layer_uses_norm(g)) {
        for (size_t b = 0; b < B; ++b)
            for (size_t j = 0; j < D; ++j) dst[at + b * D + j] += q->norm_errors[at + b * D + j]; /* Backward_Pass__Identity, :1084-1108 */
    } else bwd_fc(n, t, B, q->H, D, q->neuron_errors, n->parameters + g->first_connection_index, dst);
}

/* Backward_Pass__Gradient__Residual__FC: :822-950 - delta of the summation -> input side: dX = delta * W into the
 * activation errors (block's first layer: into the normalisation errors, or nothing when it is not normalised),
 * then act' on the input-side activation, then [BN backward] over the fan-in wide normalised units. */
static void bwd_gradient_residual_fc(myea_oracle_net *n, size_t li, size_t t, size_t B)
{
    const myea_layer_desc *l = &n->d.layers[li];
    olayer *o = &n->L[li];
    size_t In = o->In, Bmax = n->d.batch_size;
    int renorm = l->type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
    float *din;
    if (o->group == 2) din = o->af_errors;
    else if (layer_uses_norm(l)) din = o->norm_errors;
    else return;
    memset(din + t * Bmax * In, 0, Bmax * In * sizeof(float));
    bwd_fc(n, t, B, o->H, In, o->neuron_errors, n->parameters + l->first_connection_index, din);
    const float *prev_out = layer_outputs(n, o->prev);
    if (o->group == 2 && is_ind_rnn(l)) {
        /* :865-880: through the recurrence; what the member hands on is its dAFs (the AF errors keep the step's own share).
         * Nothing undoes the dropout or the k-sparse filter on the way back. */
        bwd_df_ind_rnn(n, t, B, In, n->parameters + l->first_connection_index + o->H * In, l->type_activation_function, l->activation_steepness,
                       o->unit_af, o->unit_steep, o->pre_afs, o->values, din, o->dafs, o->af_errors);
        din = o->dafs;
    } else if (o->group == 2) {
        const float *pre_af = layer_uses_norm(l) ? o->normalizes : prev_out; /* ptr_array_pre_activation_functions */
        bwd_df(n, t, B, In, l->type_activation_function, l->activation_steepness, o->unit_af, o->unit_steep, pre_af, o->values, din, o->af_errors);
    }
    if (layer_uses_norm(l)) bwd_bn(n, renorm, li, t, B, In, prev_out /* ptr_array_pre_normalization */, din, o->norm_errors);
}

/* Backward_Pass__Residual__Block: :351-452 - the residual layer's errors reach the block's last member through the
 * (cropped) shortcut add, then [block-level BN backward], copied into the member's delta. */
static void bwd_residual_block_to_last(myea_oracle_net *n, size_t ri, size_t t, size_t B, float *dst)
{
    const myea_layer_desc *r = &n->d.layers[ri];
    olayer *o = &n->L[ri];
    size_t D = o->NH, Bmax = n->d.batch_size, at = t * Bmax * D;
    float *tmp = dst;
    if (layer_uses_norm(r)) { tmp = o->norm_errors; memset(tmp + at, 0, Bmax * D * sizeof(float)); }
    bwd_residual_shortcut(n, t, B, o->H, D, o->pad, o->af_errors, tmp);
    /* Backward_Pass__Dropout__ShakeDrop (NN/Neural_Network__Backward_Pass__Loop.cpp:433-443, 1050-1078): the perturbed examples'
     * deltas times fresh U(0, 1) draws, one per value */
    if (r->type_dropout == MYEA_DROPOUT_SHAKEDROP) {
        const size_t T = n->d.number_recurrent_depth;
        const float *mask = o->noise + t * Bmax, *beta = o->noise + T * Bmax + T * Bmax * D + t * Bmax * D;
        for (size_t b = 0; b < B; ++b)
            if (mask[b] != 0.f)
                for (size_t j = 0; j < D; ++j) tmp[at + b * D + j] *= beta[b * D + j];
    }
    if (layer_uses_norm(r)) {
        int renorm = r->type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
        bwd_bn(n, renorm, ri, t, B, D, layer_outputs(n, ri + r->block_depth), tmp, o->norm_errors);
        memcpy(dst + at, o->norm_errors + at, Bmax * D * sizeof(float));
    }
}

/* Backward_Pass__Gradient__Residual: :711-729 with Backward_Pass__Gradient__Residual__Layer :731-820 - members from the
 * last to the first: zero the member's delta, pull it from its consumer, reduce it to the input side. */
static void bwd_gradient_residual(myea_oracle_net *n, size_t ri, size_t B)
{
    const myea_layer_desc *r = &n->d.layers[ri];
    size_t Bmax = n->d.batch_size, T = n->d.number_recurrent_depth, last = ri + r->block_depth;
    /* Recurrent__Backward_Pass__Gradient__Residual__Layer (NN/Neural_Network__Recurrent_Backward_Pass__OpenMP.cpp:885-1001): the
     * member's delta is pulled from its consumer over all time steps first (descending for dense, pooling and residual
     * consumers, ascending for an LSTM consumer), then the member reduces it */
    for (size_t li = last; li > ri; --li) {
        olayer *o = &n->L[li];
        const myea_layer_desc *l = &n->d.layers[li];
        const int pooling = is_pooling(l), lstm = l->type_layer == MYEA_LAYER_LSTM;
        float *delta = (pooling || lstm) ? o->af_errors : o->neuron_errors;   /* Layer::ptr_array_derivative_outputs of the member */
        memset(delta, 0, T * Bmax * o->H * sizeof(float));
        if (li != last && n->d.layers[li + 1].type_layer == MYEA_LAYER_LSTM) {
            for (size_t t = 0; t < T; ++t) bwd_lstm_to_previous(n, li + 1, t, B, delta);
        } else for (size_t t = T; t-- > 0;) {
            if (li == last) bwd_residual_block_to_last(n, ri, t, B, delta);
            else if (is_pooling(&n->d.layers[li + 1])) bwd_pooling_to_previous(n, li + 1, t, B, delta);   /* :753-758, :767-772 */
            else bwd_residual_fc_to_previous(n, li + 1, t, B, delta);
        }
        if (lstm) bwd_lstm_layer(n, li, B);
        else if (!pooling) for (size_t t = T; t-- > 0;) bwd_gradient_residual_fc(n, li, t, B);   /* a pooling member has nothing of its own to reduce (:802-804) */
    }
}

/* FF__Backward_Pass_Batch: NN/Neural_Network__Backward_Pass__OpenMP.cpp:24-155.
 * RNN__Backward_Pass_Batch: NN/Neural_Network__Recurrent_Backward_Pass__OpenMP.cpp:24-181 (FC
 * consumers iterate t descending).  The input layer's delta is never computed.  The walk goes from consumer
 * `gi` to its producer `li = previous_connected_layers[0]`; a producer collects from every consumer in
 * next_connected_layers (a layer in front of a residual block feeds the shortcut AND the block's first member);
 * after a residual layer's block has been processed the walk resumes from the residual layer itself (:117-120). */
int myea_oracle_backward_pass(myea_oracle_net *n, size_t B)
{
    if (!n) return MYEA_E_INVALID;
    if (B > n->d.batch_size) return MYEA_E_BATCH;
    if (n->state != MYEA_STATE_TRAINING) return MYEA_E_STATE;
    size_t T = n->d.number_recurrent_depth, Bmax = n->d.batch_size;
    for (size_t gi = n->d.n_layers - 1; gi != 1; --gi) {
        size_t li = n->L[gi].prev;
        const myea_layer_desc *cur = &n->d.layers[li];
        olayer *o = &n->L[li];
        float *dst = layer_derivative_outputs(n, li);
        memset(dst, 0, T * Bmax * o->H * sizeof(float));
        /* next_connected_layers (Organize__Next_Layers_Connected, NN/Neural_Network.cpp:59-102) */
        size_t consumers[2], nc = 0;
        consumers[nc++] = cur->type_layer == MYEA_LAYER_RESIDUAL ? li + cur->block_depth + 1 : li + 1;
        if (n->d.layers[consumers[0]].type_layer == MYEA_LAYER_RESIDUAL) consumers[nc++] = consumers[0] + 1;
        for (size_t c = 0; c < nc; ++c) {
            size_t ci = consumers[c];
            const myea_layer_desc *next = &n->d.layers[ci];
            if (is_dense(next)) {
                if (n->L[ci].group) for (size_t tt = T; tt-- > 0;) bwd_residual_fc_to_previous(n, ci, tt, B, dst);
                else for (size_t tt = T; tt-- > 0;)
                    bwd_fc(n, tt, B, n->L[ci].H, o->H, n->L[ci].neuron_errors, n->parameters + next->first_connection_index, dst);
            } else if (next->type_layer == MYEA_LAYER_LSTM) {
                for (size_t tt = 0; tt < T; ++tt) bwd_lstm_to_previous(n, ci, tt, B, dst);
            } else if (next->type_layer == MYEA_LAYER_RESIDUAL) {
                for (size_t tt = T; tt-- > 0;) bwd_residual_shortcut(n, tt, B, n->L[ci].H, o->H, n->L[ci].pad, n->L[ci].af_errors, dst);
            } else if (is_pooling(next)) {
                for (size_t tt = 0; tt < T; ++tt) bwd_pooling_to_previous(n, ci, tt, B, dst);
            } else return MYEA_E_UNSUPPORTED;
        }
        if (is_dense(cur)) {
            for (size_t tt = T; tt-- > 0;) bwd_gradient_fc(n, li, tt, B);
        } else if (cur->type_layer == MYEA_LAYER_LSTM) {
            bwd_lstm_layer(n, li, B);
        } else if (cur->type_layer == MYEA_LAYER_RESIDUAL) {
            bwd_gradient_residual(n, li, B);
            gi = li + 1;
        } else if (is_pooling(cur)) {
            /* a pooling layer has no gradient of its own (NN/Neural_Network__Backward_Pass__Loop.cpp:184-185) */
        } else return MYEA_E_UNSUPPORTED;
    }
    return MYEA_OK;
}

/* ------------------------------------------------------------------------------------------- */
/* Update_Derivative_Weight */

/* Update_Derivative_Weight__FC (7-arg): NN/Neural_Network__Update_Derivative_Weight__OpenMP.cpp:178-216;
 * Update_Derivative_Weight__Bias: :218-242.  dW += delta^T X; db += column sums. */
static void dw_fc(myea_oracle_net *n, size_t t, size_t B, size_t In, size_t Out, const float *x, const float *delta, float *dw)
{
    size_t Bmax = n->d.batch_size;
    const float *xt = x + Bmax * In * t, *dt = delta + Bmax * Out * t;
    long o;
    /* parallel over output rows: same per-element summation order as the serial loop */
#pragma omp parallel for schedule(static) num_threads(n->threads)
    for (o = 0; o < (long)Out; ++o) {
        float *row = dw + (size_t)o * In;
        for (size_t b = 0; b < B; ++b) {
            float e = dt[b * Out + (size_t)o];
            const float *xi = xt + b * In;
            for (size_t i = 0; i < In; ++i) row[i] += e * xi[i];
        }
    }
}

static void dw_bias(myea_oracle_net *n, size_t t, size_t B, size_t Out, const float *delta, float *db)
{
    const float *dt = delta + n->d.batch_size * Out * t;
    for (size_t b = 0; b < B; ++b)
        for (size_t o = 0; o < Out; ++o) db[o] += dt[b * Out + o];
}

/* FF__Update_Derivative_Weight_Batch: :24-59; RNN variant:
 * NN/Neural_Network__Recurrent_Update_Derivative_Weight__OpenMP.cpp:24-166 (per layer, t ascending).
 * X is Layer::ptr_array_pre_summations = the previous layer's (post-dropout) outputs. */
int myea_oracle_update_derivative_weight(myea_oracle_net *n, size_t B, size_t first, size_t end)
{
    if (!n || first < 1 || end > n->d.n_layers || first > end) return MYEA_E_INVALID;
    if (B > n->d.batch_size) return MYEA_E_BATCH;
    size_t T = n->d.number_recurrent_depth;
    for (size_t li = first; li < end; ++li) {
        const myea_layer_desc *l = &n->d.layers[li];
        if (l->type_layer == MYEA_LAYER_RESIDUAL || is_pooling(l)) continue;
        if (l->type_layer == MYEA_LAYER_LSTM) { dw_lstm(n, li, B); continue; }
        if (!is_dense(l)) return MYEA_E_UNSUPPORTED;
        olayer *o = &n->L[li];
        /* Layer::ptr_array_pre_summations (NN/Neural_Network__Ordered.cpp:96-141): inside a residual block the operand
         * the weights were applied to - the layer's own activation values, or for the block's first layer its normalised
         * input / the shortcut source's output */
        const float *x = layer_outputs(n, o->prev);
        if (o->group == 2) x = o->values;
        else if (o->group == 1 && layer_uses_norm(l)) x = o->normalizes;
        for (size_t t = 0; t < T; ++t) {
            dw_fc(n, t, B, o->In, o->H, x, o->neuron_errors, n->gradient + l->first_connection_index);
            if (layer_uses_bias(l)) dw_bias(n, t, B, o->H, o->neuron_errors, n->gradient + l->first_bias_connection_index);
            /* Update_Derivative_Weight__FC_Ind_RNN (NN/Neural_Network__Recurrent_Update_Derivative_Weight__Loop.cpp:461-483),
             * from the second time step on: du += AF[t-1] * dAF[t] */
            if (t != 0 && is_ind_rnn(l) && o->group != 1) {   /* a block's first member owns no recurrent unit (tmp_AF_size == 0) */
                size_t Bmax = n->d.batch_size, H = o->group ? o->AH : o->H;
                float *du = n->gradient + l->first_connection_index + o->H * o->In;
                for (size_t b = 0; b < B; ++b)
                    for (size_t j = 0; j < H; ++j) du[j] += o->values[Bmax * H * (t - 1) + b * H + j] * o->dafs[Bmax * H * t + b * H + j];
            }
        }
    }
    return MYEA_OK;
}

/* Update_Parameter__iRPROP_minus__Loop: NN/Neural_Network__iRPROP_minus.cpp:21-67.  Same slope sign: the step grows (capped) and
 * is taken; opposite sign: the step shrinks (floored), the slope is forgotten and - the sign of a forgotten slope being 0 - the
 * weight stays; otherwise the step is taken as it is. */
static float irprop_sign(float x) { return x > 0.f ? 1.f : (x < 0.f ? -1.f : 0.f); }

void myea_oracle_irprop_minus(const myea_hyper *h, size_t count, float *w, float *g, float *steps, float *slopes)
{
    for (size_t i = 0; i < count; ++i) {
        float gi = g[i], d;
        if (slopes[i] * gi > 0.f) {
            d = steps[i] * h->rprop_increase_factor;
            steps[i] = d = d < h->rprop_delta_max ? d : h->rprop_delta_max;
        } else if (slopes[i] * gi < 0.f) {
            d = steps[i] * h->rprop_decrease_factor;
            steps[i] = d = d > h->rprop_delta_min ? d : h->rprop_delta_min;
            gi = 0.f;
        } else d = steps[i];
        w[i] += -irprop_sign(gi) * d;
        slopes[i] = gi;
        g[i] = 0.f;
    }
}

/* ------------------------------------------------------------------------------------------- */
/* Update_Parameter: NN/Neural_Network.cpp:4719-4908 (merge is a no-op with one accumulator) */

/* Euclidean_Norm (Clip_Gradient): NN/Neural_Network__Regularization__Max_Norm_Constraints.cpp:48-140,
 * NN/Neural_Network__Clip_Gradient.cpp:81-94.  One global norm over all P; scale when norm >= clip. */
static void clip_gradient(myea_oracle_net *n)
{
    size_t P = n->d.total_parameters;
    float norms = 0.f;
    for (size_t i = 0; i < P; ++i) norms += n->gradient[i] * n->gradient[i];
    norms = sqrtf(norms);
    if (norms >= n->h.clip_gradient) {
        float s = n->h.clip_gradient / norms;
        for (size_t i = 0; i < P; ++i) n->gradient[i] *= s;
    }
}

static float clipf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* Warm_Restarts_Decay NN/Train.cpp:266-283: cosine-annealed rate from the step count BEFORE this update; at the end of a
 * cycle the optimizer is cleared, the cycle lengthens and its maximum rate decays */
static float warm_restarts_decay(myea_oracle_net *n)
{
    myea_hyper *h = &n->h;
    float lr = h->warm_restarts_minimum_learning_rate + 0.5f * (h->warm_restarts_maximum_learning_rate - h->warm_restarts_minimum_learning_rate)
                   * (1.f + cosf(h->optimizer_time_step / h->warm_restarts_T_i * 3.14159265358979323846f));
    if (h->optimizer_time_step >= h->warm_restarts_T_i) {
        clear_optimizer(n);
        h->warm_restarts_T_i *= h->warm_restarts_multiplier;
        h->warm_restarts_maximum_learning_rate *= h->warm_restarts_decay_learning_rate;
        if (h->warm_restarts_maximum_learning_rate < h->warm_restarts_minimum_learning_rate) h->warm_restarts_maximum_learning_rate = h->warm_restarts_minimum_learning_rate;
    }
    return lr;
}

/* Euclidean_Norm NN/Neural_Network__Regularization__Max_Norm_Constraints.cpp:48-82 */
static void max_norm_vector(float *v, size_t n, float max_norm)
{
    float s = 0.f;
    for (size_t i = 0; i < n; ++i) s += v[i] * v[i];
    s = sqrtf(s);
    if (s >= max_norm) { float r = max_norm / s; for (size_t i = 0; i < n; ++i) v[i] *= r; }
}

/* Update_Weight_Regularization__Max_Norm_Constraints NN/Neural_Network__Regularization__Max_Norm_Constraints.cpp:140-529 with
 * (start, end) = (0, total_weights): every fully-connected neuron's incoming weight vector (hidden and output layers) is
 * rescaled onto the ball of radius max_norm; for an LSTM block the same is done per weight segment (per cell: cell-input
 * feed-forward and recurrent; per block: the three gates' feed-forward, recurrent and peephole vectors).  The LSTM tests
 * are `first index > start`, so a segment that begins at flat index 0 is left alone (:184, :197, ... as written). */
static void max_norm_segment(myea_oracle_net *n, size_t first, size_t len, int strict)
{
    if (strict && first == 0) return;
    max_norm_vector(n->parameters + first, len, n->h.regularization__max_norm_constraints);
}

static int max_norm_constraints(myea_oracle_net *n)
{
    for (size_t li = 1; li < n->d.n_layers; ++li) {
        const myea_layer_desc *l = &n->d.layers[li];
        if (l->type_layer == MYEA_LAYER_RESIDUAL || is_pooling(l)) continue;
        if (is_dense(l)) {   /* neuron units: an independently recurrent layer's self weights are not among them */
            for (size_t o = 0; o < n->L[li].H; ++o) max_norm_segment(n, l->first_connection_index + o * n->L[li].In, n->L[li].In, 0);
        } else if (l->type_layer == MYEA_LAYER_LSTM) {
            for (int dir = 0; dir < (l->use_bidirectional ? 2 : 1); ++dir) {
                const olstm *q = &n->L[li].lstm[dir];
                for (size_t k = 0; k < q->K; ++k) {
                    for (size_t j = 0; j < q->cpb; ++j) {
                        max_norm_segment(n, lstm_z_in(l, q, k, j), q->In, 1);
                        max_norm_segment(n, lstm_z_rec(l, q, k, j), q->C, 1);
                    }
                    for (int g = 0; g < 3; ++g) max_norm_segment(n, lstm_gate_in(l, q, k, g), q->In, 1);
                    for (int g = 0; g < 3; ++g) max_norm_segment(n, lstm_gate_rec(l, q, k, g), q->C, 1);
                    for (int g = 0; g < 3; ++g) max_norm_segment(n, lstm_peep(l, q, k, g), q->cpb, 1);
                }
            }
        } else return MYEA_E_UNSUPPORTED;
    }
    return MYEA_OK;
}

int myea_oracle_update_parameter(myea_oracle_net *n, size_t B, size_t training_size)
{
    if (!n) return MYEA_E_INVALID;
    size_t P = n->d.total_parameters, W = n->d.total_weights;
    myea_hyper *h = &n->h;
    float *g = n->gradient, *w = n->parameters;
    /* the L1 / L2 gradient terms are called with (batch size, 0, total weights) where the callee expects (start, end, batch
     * size): both loops are empty, the terms never reach the gradient (NN/Neural_Network.cpp:4729-4740 against
     * NN/Neural_Network__Regularization__L1.cpp:98-128) - nothing to do here */
    if (h->use_clip_gradient) clip_gradient(n);
    int adam_type = h->type_optimizer_function != MYEA_OPTIMIZER_GD && h->type_optimizer_function != MYEA_OPTIMIZER_IRPROP_PLUS;
    float scale = 1.f;
    if (h->use_Warm_Restarts && h->type_optimizer_function != MYEA_OPTIMIZER_IRPROP_PLUS)
        scale = warm_restarts_decay(n) / (adam_type ? h->adam_learning_rate : h->learning_rate);
    if (h->type_optimizer_function != MYEA_OPTIMIZER_IRPROP_PLUS) h->optimizer_time_step += 1.f;
    /* Normalized_Weight_Decay NN/Train.cpp:285-286 */
    float wd = h->use_normalized_weight_decay ? h->regularization__weight_decay * sqrtf((float)B / ((float)training_size * h->epoch_time_step)) : h->regularization__weight_decay;
    if (h->regularization__weight_decay == 0.f) wd = 0.f;   /* keeps a call without a training-set size well defined */
    switch (h->type_optimizer_function) {
    case MYEA_OPTIMIZER_GD: {
        /* NN/Neural_Network__Gradient_Descent.cpp:22-159, NN/Neural_Network__Gradient_Descent_Momentum.cpp:22-62,
         * NN/Neural_Network__Nesterov_Accelerated_Gradient.cpp:22-64 */
        float lr = scale * h->learning_rate, mu = h->learning_momentum;
        wd *= scale;
        float *dprev = n->opt[MYEA_STATE_PREVIOUS_DELTA];
        long i;
        /* elementwise: the thread split does not change any result (the reference's __OpenMP variants do the same) */
#pragma omp parallel for schedule(static) num_threads(n->threads)
        for (i = 0; i < (long)P; ++i) {
            float reg = (wd != 0.f) ? ((size_t)i < W ? 1.f : 0.f) * wd * w[i] : 0.f;
            if (mu == 0.f) {
                if (wd != 0.f) w[i] -= lr * g[i] + reg; else w[i] -= lr * g[i];
            } else if (!h->use_Nesterov) {
                float d = dprev[i] = lr * g[i] + mu * dprev[i];
                if (wd != 0.f) w[i] -= d + reg; else w[i] -= d;
            } else {
                float d = dprev[i] = lr * g[i] + mu * dprev[i];
                if (wd != 0.f) w[i] -= mu * d - lr * g[i] + reg; else w[i] -= mu * d - lr * g[i]; /* sign as written, :48,59 */
            }
            g[i] = 0.f;
        }
        break;
    }
    case MYEA_OPTIMIZER_ADAM:
    case MYEA_OPTIMIZER_AMSGRAD:
    case MYEA_OPTIMIZER_ADABOUND:
    case MYEA_OPTIMIZER_AMSBOUND:
    case MYEA_OPTIMIZER_NOSADAM: {
        /* NN/Neural_Network__Adam.cpp:43-97, NN/Neural_Network__AMSGrad.cpp:43-105, NN/Neural_Network__AdaBound.cpp:43-110,
         * NN/Neural_Network__AMSBound.cpp:43-110, NN/Neural_Network__NosAdam.cpp:43-100 */
        uint32_t kind = h->type_optimizer_function;
        float lr = scale * h->adam_learning_rate, b1 = h->adam_beta1, b2 = h->adam_beta2, eps = h->adam_epsilon, ts = h->optimizer_time_step;
        /* every operand is a T_ = float there (NN/Neural_Network__Adam.cpp:58): float pow and sqrt, product first, then the quotient */
        float lr_t = h->use_adam_bias_correction ? lr * sqrtf(1.f - powf(b2, ts)) / (1.f - powf(b1, ts)) : lr;
        float lo = scale * h->learning_rate_final * (1.f - 1.f / (h->learning_gamma * ts + 1.f));
        float hi = scale * h->learning_rate_final * (1.f + 1.f / (h->learning_gamma * ts));
        float b2v = b2;   /* the decay applied to the second moment */
        if (kind == MYEA_OPTIMIZER_NOSADAM) {
            float pg = powf(ts, -h->adam_gamma);
            b2v = h->adam_previous_beta2 / (h->adam_previous_beta2 + pg);
            h->adam_previous_beta2 += pg;
        }
        float *m = n->opt[MYEA_STATE_FIRST_MOMENT], *v = n->opt[MYEA_STATE_SECOND_MOMENT], *vh = n->opt[MYEA_STATE_SECOND_MOMENT_HAT];
        long i;
#pragma omp parallel for schedule(static) num_threads(n->threads)
        for (i = 0; i < (long)P; ++i) {
            float gi = g[i];
            float mi = m[i] = b1 * m[i] + (1.f - b1) * gi;
            float vi = v[i] = b2v * v[i] + (1.f - b2v) * gi * gi;
            float reg = (wd != 0.f) ? ((size_t)i < W ? 1.f : 0.f) * wd * w[i] : 0.f;
            float step;
            if (kind == MYEA_OPTIMIZER_ADAM || kind == MYEA_OPTIMIZER_NOSADAM) step = lr_t * mi / (sqrtf(vi) + eps);
            else if (kind == MYEA_OPTIMIZER_AMSGRAD) {
                float hh = vh[i] = vh[i] > vi ? vh[i] : vi;
                step = lr_t * mi / (sqrtf(hh) + eps);
            } else if (kind == MYEA_OPTIMIZER_AMSBOUND) {
                float hh = vh[i] = vh[i] > vi ? vh[i] : vi;
                step = clipf(lr_t / (sqrtf(hh) + eps), lo, hi) * mi;
            } else step = clipf(lr_t / (sqrtf(vi) + eps), lo, hi) * mi;
            if (wd != 0.f) w[i] -= step + reg; else w[i] -= step;
            g[i] = 0.f;
        }
        break;
    }
    case MYEA_OPTIMIZER_IRPROP_PLUS: {
        /* NN/Neural_Network__iRPROP_plus.cpp:28-117: sign-based steps; a sign change shrinks the step, takes the last weight change
         * back when the loss got worse, and forgets the slope */
        int worse = h->loss_rprop > h->previous_loss_rprop;
        float *dprev = n->opt[MYEA_STATE_PREVIOUS_DELTA], *st = n->opt[MYEA_STATE_PREVIOUS_STEPS], *gp = n->opt[MYEA_STATE_PREVIOUS_DERIVATIVES];
        for (size_t i = 0; i < P; ++i) {
            float gi = g[i], s = gp[i] * gi;
            if (s > 0.f) {
                float d = st[i] * h->rprop_increase_factor;
                st[i] = d = d < h->rprop_delta_max ? d : h->rprop_delta_max;
                dprev[i] = -sign_f(gi) * d;
                w[i] += dprev[i];
                gp[i] = gi;
            } else if (s < 0.f) {
                float d = st[i] * h->rprop_decrease_factor;
                st[i] = d > h->rprop_delta_min ? d : h->rprop_delta_min;
                if (worse) w[i] -= dprev[i];
                gp[i] = 0.f;
            } else {
                dprev[i] = -sign_f(gi) * st[i];
                w[i] += dprev[i];
                gp[i] = gi;
            }
            g[i] = 0.f;
        }
        break;
    }
    default:
        h->optimizer_time_step -= 1.f;
        return MYEA_E_UNSUPPORTED;
    }
    if (h->regularization__max_norm_constraints != 0.f) { int rc = max_norm_constraints(n); if (rc != MYEA_OK) return rc; }
    /* Update_Weight_Regularization__Constraint_Recurrent_Weight (NN/Neural_Network__Regularization__Constraint_Recurrent_Weight.cpp:
     * 289-333): hidden layers only; the self weights of an independently recurrent layer clipped to its bounds */
    for (size_t li = 1; li + 1 < n->d.n_layers; ++li) {
        const myea_layer_desc *l = &n->d.layers[li];
        if (!is_ind_rnn(l) || n->L[li].group == 1 || (l->constraint_recurrent_weight_lower_bound == 0.f && l->constraint_recurrent_weight_upper_bound == 0.f)) continue;
        float *u = n->parameters + l->first_connection_index + n->L[li].H * n->L[li].In;   /* one per recurrent activation unit */
        for (size_t j = 0; j < (n->L[li].group ? n->L[li].AH : n->L[li].H); ++j) u[j] = clipf(u[j], l->constraint_recurrent_weight_lower_bound, l->constraint_recurrent_weight_upper_bound);
    }
    return MYEA_OK;
}

int myea_oracle_reset_loss(myea_oracle_net *n) { if (!n) return MYEA_E_INVALID; memset(&n->loss, 0, sizeof(n->loss)); return MYEA_OK; }
int myea_oracle_get_loss(myea_oracle_net *n, myea_loss_state *s) { if (!n || !s) return MYEA_E_INVALID; *s = n->loss; return MYEA_OK; }

const float *myea_oracle_tensor(myea_oracle_net *n, size_t li, int kind, size_t *count)
{
    if (!n || li >= n->d.n_layers) return NULL;
    olayer *o = &n->L[li];
    size_t T = n->d.number_recurrent_depth, full = T * n->d.batch_size * o->H, th = T * o->NH;
    const float *p = NULL; size_t c = full;
    switch (kind) {
    case MYEA_TENSOR_OUTPUTS: p = layer_outputs(n, li); break;
    case MYEA_TENSOR_SUMMATIONS: p = o->summations; break;
    case MYEA_TENSOR_ERRORS: p = (n->d.layers[li].type_layer == MYEA_LAYER_RESIDUAL || is_pooling(&n->d.layers[li])) ? o->af_errors : o->neuron_errors; break;
    case MYEA_TENSOR_NORM_HATS: p = o->hats; c = T * n->d.batch_size * o->NH; break;
    case MYEA_TENSOR_DROPOUT_NOISE:
        p = o->noise;
        if (n->d.layers[li].type_layer == MYEA_LAYER_RESIDUAL) c = T * n->d.batch_size * (1 + 2 * o->NH);
        else c = T * n->d.batch_size * o->AH;
        break;
    case MYEA_TENSOR_INPUT_SIDE_ERRORS:
        if (o->group == 2) p = layer_uses_norm(&n->d.layers[li]) ? o->norm_errors : (is_ind_rnn(&n->d.layers[li]) ? o->dafs : o->af_errors);
        else if (o->group == 1 && layer_uses_norm(&n->d.layers[li])) p = o->norm_errors;
        c = T * n->d.batch_size * o->In;
        break;
    case MYEA_TENSOR_NORM_MEANS: p = o->means; c = th; break;
    case MYEA_TENSOR_NORM_VARIANCES: p = o->variances; c = th; break;
    case MYEA_TENSOR_NORM_MEANS_AVERAGES: p = o->means_averages; c = th; break;
    case MYEA_TENSOR_NORM_VARIANCES_AVERAGES: p = o->variances_averages; c = th; break;
    default: break;
    }
    if (o->lstm) {
        int backward = (kind & MYEA_TENSOR_DIRECTION_BACKWARD) != 0;
        if (backward && !n->d.layers[li].use_bidirectional) { if (count) *count = 0; return NULL; }
        olstm *q = &o->lstm[backward];
        kind &= ~MYEA_TENSOR_DIRECTION_BACKWARD;
        size_t cc = T * n->d.batch_size * q->C, kk = T * n->d.batch_size * q->K;
        int group = (kind >> MYEA_TENSOR_LSTM_NORM_GROUP_SHIFT) & 15;   /* 1 + the group of normalised units, or 0 */
        kind &= ~(15 << MYEA_TENSOR_LSTM_NORM_GROUP_SHIFT);
        if (group) {
            p = NULL;
            if (q->norm && group <= 9) {
                obn *bn = &q->nrm[group - 1];
                float *deltas[9] = {q->dz_in, q->dz_rec, q->dc, q->di_in, q->di_rec, q->df_in, q->df_rec, q->do_in, q->do_rec};
                size_t full_g = T * n->d.batch_size * bn->H, th_g = T * bn->H;
                switch (kind) {
                case MYEA_TENSOR_NORM_HATS: p = bn->hats; c = full_g; break;
                case MYEA_TENSOR_NORM_MEANS: p = bn->means; c = th_g; break;
                case MYEA_TENSOR_NORM_VARIANCES: p = bn->variances; c = th_g; break;
                case MYEA_TENSOR_NORM_MEANS_AVERAGES: p = bn->means_averages; c = th_g; break;
                case MYEA_TENSOR_NORM_VARIANCES_AVERAGES: p = bn->variances_averages; c = th_g; break;
                case MYEA_TENSOR_ERRORS: p = deltas[group - 1]; c = full_g; break;
                default: break;
                }
            }
            if (count) *count = p ? c : 0;
            return p;
        }
        switch (kind) {
        case MYEA_TENSOR_LSTM_CELL_OUTPUT: p = q->h; c = cc; break;
        case MYEA_TENSOR_ERRORS: p = o->af_errors; c = cc; break;
        case MYEA_TENSOR_LSTM_DELTA_CELL_OUTPUT: p = q->dh; c = cc; break;
        case MYEA_TENSOR_LSTM_CELL_INPUT: p = q->z; c = cc; break;
        case MYEA_TENSOR_LSTM_CELL_STATE: p = q->c; c = cc; break;
        case MYEA_TENSOR_LSTM_INPUT_GATE: p = q->gi; c = kk; break;
        case MYEA_TENSOR_LSTM_FORGET_GATE: p = q->gf; c = kk; break;
        case MYEA_TENSOR_LSTM_OUTPUT_GATE: p = q->go; c = kk; break;
        case MYEA_TENSOR_LSTM_DELTA_CELL_INPUT: p = q->dz; c = cc; break;
        case MYEA_TENSOR_LSTM_DELTA_CELL_STATE: p = q->dc; c = cc; break;
        case MYEA_TENSOR_LSTM_DELTA_INPUT_GATE: p = q->di; c = kk; break;
        case MYEA_TENSOR_LSTM_DELTA_FORGET_GATE: p = q->df; c = kk; break;
        case MYEA_TENSOR_LSTM_DELTA_OUTPUT_GATE: p = q->dgo; c = kk; break;
        default: break;
        }
    }
    if (count) *count = p ? c : 0;
    return p;
}
