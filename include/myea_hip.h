/* myea_hip.h — C ABI of the MI355X (gfx950) training hot path.
 *
 * This is the boundary a host-side `Neural_Network` plugs into where the
 * reference plugs in its CUDA object (`Set__CUDA` / `Initialize__CUDA` /
 * `Copy__Host_To_Device`, Header_Files/Neural_Network/Data.hpp:3111-3196,
 * Source_Files/Neural_Network/Neural_Network.cpp:2852-2912).  Every entry point
 * names the reference member function it replaces.
 *
 * Conventions
 *   - plain C, plain pointers and sizes; no C++/torch types cross this line;
 *   - every function returns 0 on success or a negative MYEA_E_* code and never
 *     aborts; myea_hip_last_error() returns the text of the last failure on
 *     the calling thread (the reference prints and returns `false`);
 *   - one net = one training stream; calls on one net must come from one host
 *     thread at a time (the reference has the same rule: its step functions are
 *     orphaned OpenMP constructs entered by a whole thread team);
 *   - all arithmetic is IEEE fp32 (`T_ = float`, Common_Library/include/
 *     Configuration/DTypes.hpp:20-32); indices are 64-bit; masks are bytes.
 *   - tensors of a layer are row-major [T][batch_size][units] exactly as in the
 *     reference (Neural_Network__Backward_Pass__OpenMP.cpp:1055-1072);
 *   - the flat parameter vector keeps the reference order
 *     [weights | biases | normalisation scales | normalisation shifts]
 *     (Neural_Network__Compile.cpp:556-665, Neural_Network__Allocate.cpp:2378-2406).
 */
#ifndef MYEA_HIP_H
#define MYEA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- enums: numeric values are the reference's (Common_Library/include/Enums) ---- */

/* Enum_Type_Layer.hpp */
enum {
    MYEA_LAYER_NONE = 0,
    MYEA_LAYER_FULLY_CONNECTED = 4,
    MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT = 5,  /* h[t] = AF(W x[t] + b + u * h[t-1]), one self weight per unit */
    MYEA_LAYER_AVERAGE_POOLING = 1,
    MYEA_LAYER_LSTM = 8,
    MYEA_LAYER_MAX_POOLING = 9,
    MYEA_LAYER_RESIDUAL = 10
};

/* Enum_Type_Networks.hpp */
enum { MYEA_NETWORK_FEEDFORWARD = 3, MYEA_NETWORK_RECURRENT = 4 };

/* Enum_Type_Activation_Functions.hpp */
enum {
    MYEA_AF_NONE = 0, MYEA_AF_COSINE = 1, MYEA_AF_COSINE_SYMMETRIC = 2, MYEA_AF_ELU = 3,
    MYEA_AF_ELLIOT = 4, MYEA_AF_ELLIOT_SYMMETRIC = 5, MYEA_AF_GAUSSIAN = 6,
    MYEA_AF_GAUSSIAN_STEPWISE = 7, MYEA_AF_GAUSSIAN_SYMMETRIC = 8, MYEA_AF_ISRU = 9,
    MYEA_AF_ISRLU = 10, MYEA_AF_LINEAR = 11, MYEA_AF_LINEAR_PIECE = 12,
    MYEA_AF_LINEAR_PIECE_SYMMETRIC = 13, MYEA_AF_LEAKY_RELU = 14, MYEA_AF_PARAMETRIC_RELU = 15,
    MYEA_AF_RELU = 16, MYEA_AF_SELU = 17, MYEA_AF_SIGMOID = 18, MYEA_AF_SINE = 19,
    MYEA_AF_SIGMOID_STEPWISE = 20, MYEA_AF_SINE_SYMMETRIC = 21, MYEA_AF_SOFTMAX = 22,
    MYEA_AF_TANH = 23, MYEA_AF_TANH_STEPWISE = 24, MYEA_AF_THRESHOLD = 25,
    MYEA_AF_THRESHOLD_SYMMETRIC = 26, MYEA_AF_LENGTH = 27
};

/* Enum_Type_Optimizer_Functions.hpp */
enum {
    MYEA_OPTIMIZER_NONE = 0, MYEA_OPTIMIZER_ADABOUND = 1, MYEA_OPTIMIZER_ADAM = 2,
    MYEA_OPTIMIZER_AMSBOUND = 4, MYEA_OPTIMIZER_AMSGRAD = 5, MYEA_OPTIMIZER_GD = 6,
    MYEA_OPTIMIZER_IRPROP_MINUS = 7,   /* myea_hip_optimizer_update only: the reference's Update_Parameter has no case for it
                                        * (Neural_Network.cpp:4770-4821) and neither has myea_hip_update_parameter */
    MYEA_OPTIMIZER_IRPROP_PLUS = 8, MYEA_OPTIMIZER_NOSADAM = 9
};

/* Enum_Type_Layer_Dropout.hpp */
enum {
    MYEA_DROPOUT_NONE = 0, MYEA_DROPOUT_BERNOULLI = 2, MYEA_DROPOUT_BERNOULLI_INVERTED = 3,
    MYEA_DROPOUT_GAUSSIAN = 4, /* training state: y *= N(1, dropout_values[0]) per (example, unit); dropout_values[0] = p / (1 - p) */
    MYEA_DROPOUT_SHAKEDROP = 5, /* residual layers only: with probability dropout_values[0] an example's block output is multiplied,
                                  * value by value, by U(-1, 1) draws going forward and its delta by U(0, 1) draws going back;
                                  * outside the training state the block output is scaled by 1 - dropout_values[0] */
    MYEA_DROPOUT_UOUT = 6,     /* training state: y += y * U(-dropout_values[0], dropout_values[0]) per (example, unit) */
    MYEA_DROPOUT_ZONEOUT = 7   /* LSTM layers only: dropout_values[0] / [1] = zoneout probability of the cell state / the cell output */
};

/* Enum_Type_Layer_Normalization.hpp */
enum {
    MYEA_NORMALIZATION_NONE = 0, MYEA_NORMALIZATION_BATCH_NORMALIZATION = 1,
    MYEA_NORMALIZATION_BATCH_RENORMALIZATION = 2
};

/* Enum_Type_Loss_Functions.hpp (loss / accuracy) */
enum {
    MYEA_LOSS_NONE = 0, MYEA_LOSS_BIT = 1, MYEA_LOSS_CROSS_ENTROPY = 2, MYEA_LOSS_L1 = 3,
    MYEA_LOSS_L2 = 4, MYEA_LOSS_MAE = 5, MYEA_LOSS_MAPE = 6, MYEA_LOSS_ME = 9, MYEA_LOSS_MSE = 10,
    MYEA_LOSS_RMSE = 11, MYEA_LOSS_SMAPE = 12
};
enum {
    MYEA_ACCURACY_NONE = 0, MYEA_ACCURACY_CROSS_ENTROPY = 1, MYEA_ACCURACY_DIRECTIONAL = 2,
    MYEA_ACCURACY_DISTANCE = 3, MYEA_ACCURACY_R = 4, MYEA_ACCURACY_SIGN = 5
};

/* Enum_Type_State_Propagation.hpp */
enum { MYEA_STATE_INFERENCE = 0, MYEA_STATE_TRAINING = 1 };

/* ---- error codes ---- */
enum {
    MYEA_OK = 0,
    MYEA_E_INVALID = -1,      /* bad argument / descriptor */
    MYEA_E_UNSUPPORTED = -2,  /* layer / activation / optimizer not on this path */
    MYEA_E_BATCH = -3,        /* batch_size_received > batch_size (Forward_Pass__OpenMP.cpp:33-43) */
    MYEA_E_STATE = -4,        /* e.g. backward in inference mode (Backward_Pass__OpenMP.cpp:41-51) */
    MYEA_E_NOMEM = -5,
    MYEA_E_DEVICE = -6        /* HIP runtime error; text in myea_hip_last_error().  Also reported, once, by the next call that
                               * looks (Forward_Pass, synchronize, get_loss, any download or upload) after a kernel's bounded wait
                               * for another workgroup gave up - a resident LSTM time loop, a contraction whose tiles two
                               * workgroups share.  The pass that kernel belonged to is incomplete.  State the caller is left in:
                               * no Update_Parameter enqueued behind that kernel has changed parameters or optimizer vectors
                               * (the update kernels see a device-side flag), the optimizer's time step and the other scalars an
                               * update advances are back at their values before the first such update, the gradient is zero,
                               * and the network uses the plain form of that kernel from then on (one launch per time step, one
                               * workgroup per tile).  Repeat the mini-batch.  Only an optimizer clearing by a warm restart that
                               * fell on a skipped update is not taken back. */
};

/* ---- network descriptor ---- */

#define MYEA_MAX_LAYERS 64

/* One entry of `Neural_Network::ptr_array_layers` (struct Layer, Data.hpp:600-760), reduced to the
 * fields the hot path reads.  The index table is copied from the host `Layer` / `Block_unit` /
 * `Cell_unit` fields, never recomputed by the device side; myea_net_desc_layout() fills it the
 * way `Neural_Network::Compile` does for callers that have no host object. */
typedef struct myea_layer_desc {
    uint32_t type_layer;               /* MYEA_LAYER_* */
    uint32_t n_units;                  /* FC / independently recurrent: neurons.  LSTM: blocks per direction.  Input layer: inputs.
                                        * Pooling: written by myea_net_desc_layout.  Residual: unused (block_depth). */
    uint32_t n_cells_per_block;        /* LSTM only, >= 1 (Layer_Parameters::unit_parameters[1]) */
    uint32_t use_bidirectional;        /* LSTM only */
    uint32_t type_activation_function; /* FC and independently recurrent layers; MYEA_AF_* (whole layer, Set__Layer_Activation_Function) */
    float    activation_steepness;     /* same layers; Set__Layer_Activation_Steepness, default 1 */
    uint32_t type_dropout;             /* MYEA_DROPOUT_* */
    float    dropout_values[2];        /* [0]: Bernoulli = retention probability, Gaussian = p / (1 - p), Uout = beta, ShakeDrop = probability,
                                        * zoneout = cell-state probability; [1]: zoneout = cell-output probability */
    uint32_t type_normalization;       /* MYEA_NORMALIZATION_* */
    uint32_t use_layer_normalization_before_activation;
    uint32_t block_depth;              /* residual only: layers inside the block */
    /* pooling layers only (Layer::pooling_values, Assign__Layer NN/Neural_Network__Compile.cpp:51-58): kernel size,
     * stride, padding, dilation, ceil mode.  n_units of a pooling layer is an OUTPUT of myea_net_desc_layout
     * (Assign__Post__Layer :250-271). */
    uint32_t pooling_values[5];
    /* independently recurrent layers only: the clip applied to the self weights after every update, no clip when both
     * are 0 (Layer::constraint_recurrent_weight_{lower,upper}_bound,
     * NN/Neural_Network__Regularization__Constraint_Recurrent_Weight.cpp:317-333; Compile gives the layer the bounds of
     * Compute__Regularization__Constraint_Recurrent_Weight__Default, :33-75) */
    float    constraint_recurrent_weight_lower_bound;
    float    constraint_recurrent_weight_upper_bound;
    /* k-sparse filter on the layer's outputs (hidden fully-connected layers outside residual blocks): after the dropout
     * only the k_sparsity largest values of an example's row stay, the others become 0; at inference
     * size_t(alpha_sparsity * k_sparsity) stay.  0 = no filter (Layer::k_sparsity / ::alpha_sparsity, Data.hpp:733-734;
     * Sparse_K_Filter, NN/Neural_Network__K_Sparse.cpp:268-339; the backward pass does not look at the filter). */
    uint32_t k_sparsity;
    float    alpha_sparsity;
    /* index table (into the flat parameter / gradient / optimizer vectors, and the mask buffer) */
    uint64_t first_connection_index;       /* *Layer::ptr_first_connection_index */
    uint64_t last_connection_index;        /* *Layer::ptr_last_connection_index */
    uint64_t first_bias_connection_index;  /* Layer::first_bias_connection_index (LSTM: see Prepare__Bias__LSTM) */
    uint64_t first_normalized_unit_index;  /* offset of the layer's first Normalized_unit in the scale array */
    uint64_t first_mask_index;             /* offset of Layer::ptr_array__mask__dropout__bernoulli */
} myea_layer_desc;

typedef struct myea_net_desc {
    uint32_t type_network;            /* MYEA_NETWORK_* */
    uint32_t n_layers;                /* input layer + hidden layers + output layer */
    uint32_t number_recurrent_depth;  /* T, >= 1 */
    uint32_t batch_size;              /* allocated batch rows (Bmax) */
    uint64_t total_weights;
    uint64_t total_bias;
    uint64_t total_normalized_units;  /* 0 when no layer is normalised (no scale/shift region) */
    uint64_t total_parameters;        /* weights + bias + 2 * total_normalized_units */
    uint64_t total_mask_units;        /* bytes in the Bernoulli mask buffer */
    myea_layer_desc layers[MYEA_MAX_LAYERS];
} myea_net_desc;

/* Public training fields of `Neural_Network` (Data.hpp:2929-2970) the path reads; defaults are the
 * reference's (myea_hyper_default()). */
typedef struct myea_hyper {
    uint32_t type_optimizer_function;   /* MYEA_OPTIMIZER_* */
    uint32_t type_loss_function;        /* MYEA_LOSS_* */
    uint32_t type_accuracy_function;    /* MYEA_ACCURACY_* */
    uint32_t use_Nesterov;
    uint32_t use_adam_bias_correction;
    uint32_t use_clip_gradient;
    float learning_rate;                /* 0.01 */
    float learning_rate_final;          /* 0.1   (AdaBound) */
    float learning_momentum;            /* 0.9 */
    float learning_gamma;               /* 1e-3  (AdaBound) */
    float adam_learning_rate;           /* 1e-3 */
    float adam_beta1;                   /* 0.9 */
    float adam_beta2;                   /* 0.999 */
    float adam_epsilon;                 /* 1e-8 */
    float regularization__weight_decay; /* 0; applied to weights only (mask 1 on weights, 0 elsewhere) */
    float clip_gradient;                /* 1 */
    float accuracy_variance;            /* 0.49 */
    float bit_fail_limit;               /* 0.35 */
    float normalization_momentum_average;              /* 0.999 */
    float normalization_epsilon;                       /* 1e-5 */
    float batch_renormalization_r_correction_maximum;  /* 1 */
    float batch_renormalization_d_correction_maximum;  /* 0 */
    float optimizer_time_step;          /* 0; incremented by every update */
    uint32_t number_time_delays;        /* RNN: first k steps carry no loss */
    /* weight decay normalisation (Normalized_Weight_Decay, Train.cpp:285-286): wd * sqrt(B / (N_train * epoch_time_step)) */
    uint32_t use_normalized_weight_decay;   /* 1 */
    float epoch_time_step;                  /* 1; the caller's epoch loop increments it (Dataset.cpp:7660) */
    /* NosAdam (Neural_Network__NosAdam.cpp) */
    float adam_gamma;                       /* 0.1 */
    float adam_previous_beta2;              /* 0; running sum of t^-gamma */
    /* iRPROP+ (Neural_Network__iRPROP_plus.cpp); the caller's loop maintains the two losses (Dataset.cpp:575-579) */
    float rprop_increase_factor;            /* 1.2 */
    float rprop_decrease_factor;            /* 0.5 */
    float rprop_delta_min;                  /* 1e-6 */
    float rprop_delta_max;                  /* 50 */
    float rprop_delta_zero;                 /* 0.1: initial step, written by clear_training_arrays */
    float loss_rprop;                       /* FLT_MAX */
    float previous_loss_rprop;              /* FLT_MAX */
    /* max-norm constraint on every neuron's incoming weight vector after the update
     * (Neural_Network__Regularization__Max_Norm_Constraints.cpp:140-529); 0 = off */
    float regularization__max_norm_constraints;
    /* warm restarts (Warm_Restarts_Decay, Train.cpp:266-283) */
    uint32_t use_Warm_Restarts;             /* 0 */
    float warm_restarts_decay_learning_rate;    /* 1 */
    float warm_restarts_maximum_learning_rate;  /* 1 */
    float warm_restarts_minimum_learning_rate;  /* 1e-7 */
    float warm_restarts_T_i;                    /* 1 */
    float warm_restarts_multiplier;             /* 2 */
} myea_hyper;

/* Loss / accuracy accumulators (ptr_array_loss_values, ptr_array_number_loss,
 * ptr_array_accuracy_values[0..4], ptr_array_number_bit_fail; merged as Merge__Post__Training does,
 * Neural_Network__Merge.cpp:52-98). */
typedef struct myea_loss_state {
    double   loss_values;       /* sum of per-output loss terms since the last reset */
    uint64_t number_loss;       /* number of terms */
    double   accuracy_value;    /* ptr_array_accuracy_values[0]: hits; with the R accuracy the sum of the desired values */
    uint64_t number_bit_fail;
    /* R accuracy only (Pearson correlation over every output entry): ptr_array_accuracy_values[1..4] =
     * sum of the predicted values; then, from Compute__Accuracy__R, the numerator sum (d - mean_d)(y - mean_y)
     * and the two denominators sum (d - mean_d)^2, sum (y - mean_y)^2 */
    double   accuracy_r[4];
} myea_loss_state;

/* kinds for the optimizer-state and tensor taps */
enum {
    MYEA_STATE_PREVIOUS_DELTA = 0,       /* ptr_array_previous_delta_parameters */
    MYEA_STATE_FIRST_MOMENT = 1,         /* ptr_array_previous_biased_first_moment */
    MYEA_STATE_SECOND_MOMENT = 2,        /* ptr_array_previous_biased_second_moment */
    MYEA_STATE_SECOND_MOMENT_HAT = 3,    /* ptr_array_previous_biased_second_moment_hat */
    MYEA_STATE_PREVIOUS_STEPS = 4,       /* ptr_array_previous_steps (iRPROP) */
    MYEA_STATE_PREVIOUS_DERIVATIVES = 5  /* ptr_array_previous_derivatives_parameters (iRPROP) */
};
#define MYEA_STATE_KINDS 6
enum {
    MYEA_TENSOR_OUTPUTS = 0,        /* Layer::ptr_array_outputs (post-dropout) [T][Bmax][H] */
    MYEA_TENSOR_SUMMATIONS = 1,     /* neuron_units->ptr_array_summations */
    MYEA_TENSOR_ERRORS = 2,         /* neuron_units->ptr_array_errors (delta w.r.t. the summation);
                                       LSTM: delta of the cell outputs */
    MYEA_TENSOR_NORM_HATS = 3,      /* normalized_batch_units.ptr_array_values_hats */
    MYEA_TENSOR_NORM_MEANS = 4,     /* [T][H] batch means */
    MYEA_TENSOR_NORM_VARIANCES = 5, /* [T][H] batch sqrt(var+eps) */
    MYEA_TENSOR_NORM_MEANS_AVERAGES = 6,
    MYEA_TENSOR_NORM_VARIANCES_AVERAGES = 7,
    MYEA_TENSOR_INPUT_SIDE_ERRORS = 8,  /* member of a residual block: delta reduced to the layer's input side
                                           [Bmax][fan-in] (AF_unit errors, or the normalised units' errors when
                                           the member is normalised); absent for an un-normalised first member */
    /* LSTM taps, [T][Bmax][cells] or [T][Bmax][blocks] */
    MYEA_TENSOR_DROPOUT_NOISE = 9,      /* Gaussian / Uout dropout: the draws the last training-state forward pass used [T][Bmax][H] */
    MYEA_TENSOR_LSTM_CELL_INPUT = 16,      /* z  */
    MYEA_TENSOR_LSTM_CELL_STATE = 17,      /* c  */
    MYEA_TENSOR_LSTM_INPUT_GATE = 18,      /* i  */
    MYEA_TENSOR_LSTM_FORGET_GATE = 19,     /* f  */
    MYEA_TENSOR_LSTM_OUTPUT_GATE = 20,     /* o  */
    MYEA_TENSOR_LSTM_DELTA_CELL_INPUT = 21,
    MYEA_TENSOR_LSTM_DELTA_CELL_STATE = 22,
    MYEA_TENSOR_LSTM_DELTA_INPUT_GATE = 23,
    MYEA_TENSOR_LSTM_DELTA_FORGET_GATE = 24,
    MYEA_TENSOR_LSTM_DELTA_OUTPUT_GATE = 25,
    MYEA_TENSOR_LSTM_CELL_OUTPUT = 26,     /* h of one direction (OUTPUTS is the layer's output: the sum of both) */
    MYEA_TENSOR_LSTM_DELTA_CELL_OUTPUT = 27, /* delta of h of one direction incl. its recurrent terms (ERRORS of a
                                              bidirectional layer is the delta of the summed output, from above only) */
    MYEA_TENSOR_DIRECTION_BACKWARD = 0x100 /* OR-ed onto an LSTM kind: the time-reversed direction of a bidirectional layer */
};
/* A normalised LSTM layer owns nine groups of normalised units (Neural_Network__Allocate.cpp:2710-2790): 0 block input
 * from below, 1 block input recurrent, 2 cell state, 3 / 4 input gate, 5 / 6 forget gate, 7 / 8 output gate (from below /
 * recurrent).  (group + 1) << MYEA_TENSOR_LSTM_NORM_GROUP_SHIFT OR-ed onto NORM_HATS / NORM_MEANS / NORM_VARIANCES /
 * NORM_MEANS_AVERAGES / NORM_VARIANCES_AVERAGES selects the group's tensor ([T][Bmax][units] or [T][units]); onto ERRORS,
 * the delta of the group's input after the backward pass through its normalisation. */
#define MYEA_TENSOR_LSTM_NORM_GROUP_SHIFT 12
#define MYEA_TENSOR_LSTM_NORM_GROUP(g) (((g) + 1) << MYEA_TENSOR_LSTM_NORM_GROUP_SHIFT)

/* ---- host-side descriptor helpers (no GPU needed) ---- */

/* Defaults of the public training fields, Data.hpp:2929-2970. */
void myea_hyper_default(myea_hyper *hyper);

/* Fills the index table and the totals of `desc` from type_layer / n_units / n_cells_per_block /
 * use_bidirectional / block_depth / type_normalization, in the order `Neural_Network::Compile`
 * assigns them: Prepare__Connections__{FC,LSTM} per layer, then Prepare__Bias__{FC,LSTM} per layer
 * (Neural_Network__Compile.cpp:556-665, Neural_Network__Prepare_Connections.cpp:20-252), then the
 * normalised-unit scale/shift region (Neural_Network__Layer_Normalization.cpp:20-78,
 * Neural_Network__Allocate.cpp:2378-2462) and the mask offsets (Neural_Network.cpp:3948-3962). */
int myea_net_desc_layout(myea_net_desc *desc);

/* Layer::previous_connected_layers[0] as Organize__Previous_Layers_Connected (Neural_Network.cpp:20-57)
 * assigns it: the layer before, except that the first layer after a residual block connects to the
 * block's residual layer and the first layer inside a block to the layer the residual layer connects
 * to (the shortcut source).  0 for li == 0 or out of range. */
uint32_t myea_net_desc_previous_layer(const myea_net_desc *desc, uint32_t layer_index);

/* *Layer::ptr_number_outputs: FC neurons; LSTM blocks x cells per block; residual = max(shortcut
 * source width, width of the block's last layer) (Neural_Network__Compile.cpp:79,272-281). */
uint64_t myea_net_desc_number_outputs(const myea_net_desc *desc, uint32_t layer_index);

/* ---- life cycle: replaces Set__CUDA / Initialize__CUDA / Deinitialize__CUDA (Data.hpp:3111-3118) ---- */
typedef struct myea_hip_net myea_hip_net;

int myea_hip_create(const myea_net_desc *desc, myea_hip_net **out_net);
int myea_hip_destroy(myea_hip_net *net);
/* Launch everything on `hip_stream` (a hipStream_t; NULL = the default stream). */
int myea_hip_set_stream(myea_hip_net *net, void *hip_stream);
int myea_hip_synchronize(myea_hip_net *net);
const char *myea_hip_last_error(void);

/* ---- public-field setters: replace the `Set__*` forwarding in Train.cpp:28-90 ---- */
/* set_hyper replaces EVERY field, the ones the library itself advances included: optimizer_time_step (every update),
 * adam_previous_beta2 (NosAdam's running sum), epoch_time_step, warm_restarts_T_i and warm_restarts_maximum_learning_rate
 * (a warm restart), loss_rprop / previous_loss_rprop (Clear_Training_Arrays).  A caller that changes a setting between
 * steps starts from get_hyper, changes that field and hands the struct back - as the reference's setters change one public
 * field of the object and leave the others alone; a struct built from myea_hyper_default() would reset the optimizer's clock. */
int myea_hip_set_hyper(myea_hip_net *net, const myea_hyper *hyper);
int myea_hip_get_hyper(myea_hip_net *net, myea_hyper *hyper);
/* `type_state_propagation` (Data.hpp, Enum_Type_State_Propagation.hpp) */
int myea_hip_set_state_propagation(myea_hip_net *net, uint32_t type_state_propagation);

/* ---- parameter / state movement: replace Copy__Parameters__Host_To_Device,
 *      Copy__Parameters__Device_To_Host, Copy__Optimizer_*__{Host_To_Device,Device_To_Host}
 *      (Data.hpp:3119-3189) ---- */
int myea_hip_upload_parameters(myea_hip_net *net, const float *host_parameters, size_t count);
int myea_hip_download_parameters(myea_hip_net *net, float *host_parameters, size_t count);
int myea_hip_upload_optimizer_state(myea_hip_net *net, int kind, const float *host, size_t count);
int myea_hip_download_optimizer_state(myea_hip_net *net, int kind, float *host, size_t count);
/* `ptr_array_units_mask_dropout_bernoulli` (bool[(sum AF units) * T]), written by the caller between
 * steps exactly as the reference lets callers write its public mask buffer. */
/* Per-unit activation functions and steepnesses of one fully-connected layer: AF_unit::ptr_type_activation_function /
 * ptr_activation_steepness are per-unit arrays in the reference (Data.hpp, struct AF_unit; read per unit by
 * Forward_Pass__FC_AF and Backward_Pass__FC__DF, Neural_Network__Forward_Pass__OpenMP.cpp:4839-4868,
 * Neural_Network__Backward_Pass__OpenMP.cpp:1225-1263); its setters fill them uniformly, direct writes may not.
 * `count` = the layer's activation units (its width; inside a residual block: its fan-in).  Either array may be NULL
 * (keep the layer-wide value).  Softmax stays a layer-wide choice.  Call with both NULL to return to the layer-wide values. */
int myea_hip_set_unit_activations(myea_hip_net *net, size_t layer_index, const uint32_t *host_types, const float *host_steepness, size_t count);

int myea_hip_upload_masks(myea_hip_net *net, const uint8_t *host_masks, size_t count);
/* Zoneout masks of the LSTM layers, drawn by the caller as Dropout_Zoneout() does (Neural_Network__Dropout__Zoneout__Loop.cpp:57-87)
 * and laid out as ptr_array_cell_units_mask_dropout_zoneout (Reset__Parameters__Cell_Unit__Mask_Dropout, Neural_Network.cpp:3964-3995):
 * first the cell-STATE masks, per LSTM layer in layer order [T][cells of the layer], then - at offset T x (cells of all LSTM
 * layers) - the cell-OUTPUT masks in the same arrangement.  1 = update the unit, 0 = keep its previous value (0 on a sequence's
 * first step).  One mask per (time step, cell), shared by the batch.  `count` = 2 x T x total cells; all 1 after create.  The
 * masks act in the training state only (Neural_Network__Forward_Pass__Loop.cpp:2088-2092); the backward pass does not read them,
 * as in the reference. */
int myea_hip_upload_zoneout_masks(myea_hip_net *net, const uint8_t *host_masks, size_t count);
/* Gaussian / Uout dropout (Forward_Pass__Dropout__Gaussian / __Uout, Neural_Network__Forward_Pass__Loop.cpp:4993-5014, 5047-5068)
 * draw one random number per (time step, example, unit) inside the forward pass, strictly in the training state, from the
 * network's host generators (std::mt19937 behind std::normal_distribution / uniform_real_distribution); the backward pass never
 * sees the draws.  Two sources here:
 *  - default: a counter-based device generator (Philox 4x32-10; normal draws by Box-Muller) keyed by
 *    myea_hip_set_dropout_seed() and advanced by every training-state forward pass - same distributions, another stream;
 *  - myea_hip_upload_dropout_noise(): the caller's own draws for one layer, [T][Bmax][H] floats (`count` = T x batch_size x
 *    width), used by every following forward pass until the call is repeated with NULL / 0.  A caller that draws with the
 *    reference's generators in the reference's order gets the reference's numbers.
 * Either way MYEA_TENSOR_DROPOUT_NOISE reads back what the last forward pass used.
 * Inside a residual block the draws belong to a member's input-side activation units: [T][Bmax][fan-in].
 * ShakeDrop on a residual layer (Forward_Pass__Dropout__ShakeDrop :5016-5045, Backward_Pass__Dropout__ShakeDrop
 * Neural_Network__Backward_Pass__Loop.cpp:1050-1078; one mask per (time step, example),
 * Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:367-386) uses the same two sources; its tensor is
 * [T x batch_size masks as 0 / 1][T x batch_size x width forward draws][T x batch_size x width backward draws] with `width`
 * the block's last layer's, `count` = T x batch_size x (1 + 2 x width).  The device generator draws all three in the forward pass. */
int myea_hip_set_dropout_seed(myea_hip_net *net, uint64_t seed);
int myea_hip_upload_dropout_noise(myea_hip_net *net, size_t layer_index, const float *noise, size_t count, int noise_on_device);
/* Clear_Training_Arrays (Train.cpp:93-126) + Clear_Optimizer (Train.cpp:128-263): zero the gradient
 * vector and all optimizer state, optimizer_time_step = 0. */
int myea_hip_clear_training_arrays(myea_hip_net *net);

/* ---- the five step entry points ---- */

/* Neural_Network::Forward_Pass (Data.hpp:2896; Neural_Network__Forward_Pass__Loop.cpp:22).
 * `inputs` is [batch_size_received][T * n_inputs] row-major (the reference's array of per-example
 * row pointers, flattened); `inputs_on_device` != 0 means it is already resident in HBM. */
int myea_hip_forward_pass(myea_hip_net *net, size_t batch_size_received, const float *inputs, int inputs_on_device);

/* Neural_Network::Compute__Error (Data.hpp:1033; Neural_Network__Compute__Error__Loop.cpp:79).
 * `desired_outputs` is [batch_size_received][T * n_outputs] row-major. */
int myea_hip_compute_error(myea_hip_net *net, size_t batch_size_received, const float *desired_outputs, int desired_on_device);

/* Neural_Network::Backward_Pass (Data.hpp:1709; Neural_Network__Backward_Pass__Loop.cpp:22). */
int myea_hip_backward_pass(myea_hip_net *net, size_t batch_size_received);

/* Neural_Network::Update_Derivative_Weight (Data.hpp:2199) over layers
 * [first_layer_index, end_layer_index); the reference's callers pass (layers + 1, last). */
int myea_hip_update_derivative_weight(myea_hip_net *net, size_t batch_size_received, size_t first_layer_index, size_t end_layer_index);
/* No counterpart in the reference.  myea_hip_update_derivative_weight for callers that cannot allocate device memory
 * around the call or must not depend on buffers the library allocated (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments, same launches, same results, but every scratch buffer of
 * its kernels - the column reductions' partial sums, the split-K slabs of narrow fully-connected layers, the packed
 * weight-gradient slabs of LSTM layers - comes out of one static device array of 32 MiB that each GPU the library
 * runs on holds until the process ends.  The call allocates and frees nothing.  A network whose kernels need more
 * scratch than the array holds is rejected with MYEA_E_INVALID (the text names both sizes).  Every call on a GPU
 * shares that GPU's array: calls that overlap on one GPU (two networks on two streams) race. */
int myea_hip_update_derivative_weight_no_alloc(myea_hip_net *net, size_t batch_size_received, size_t first_layer_index, size_t end_layer_index);
/* Backward_Pass immediately followed by Update_Derivative_Weight(batch, 1, total_layers) - the two calls Dataset::Train_Batch_BP
 * issues back to back (Neural_Network/Dataset.cpp:645-658) - as one entry point.  Results are those of the two calls; knowing
 * that the weight gradients are wanted lets the library send a layer's `dW += delta^T X` along in the same launch as the
 * `dX = delta W` that hands its delta down (two 128 x 128-tiled contractions sharing the CUs keep the matrix pipe busier than
 * either alone when the batch is about a thousand rows). */
int myea_hip_backward_pass_and_update_derivative_weight(myea_hip_net *net, size_t batch_size);

/* Neural_Network::Update_Parameter (Data.hpp:849; Neural_Network.cpp:4719-4908): clip-by-global-norm
 * then the fused optimizer; zeroes the gradient. */
int myea_hip_update_parameter(myea_hip_net *net, size_t batch_size_received, size_t training_size_received);
/* Backward_Pass, Update_Derivative_Weight(batch, 1, total_layers) and Update_Parameter(batch, training size) as one entry
 * point: the tail of Train_Batch_BP (Neural_Network/Dataset.cpp:645-658) and the Update_Parameter that Dataset::Training_OpenMP
 * issues right behind it (Dataset.cpp:7652-7658).  Dataset_Mini_Batch::Training_OpenMP measures the batch's accuracy between the
 * two (Dataset__Mini_Batch.cpp:353-372): a caller of this entry point takes that measurement, which reads the weights, first.
 * Results are those of the three calls.
 * Knowing that the update follows lets the library give the weights of a fully-connected layer their optimizer step as soon as
 * their gradient is complete and the pass has no reader of them left: the memory-bound update then runs on a second stream
 * beside the matrix-pipe-bound contractions of the layers below instead of behind all of them.  That needs an update whose
 * scalars are known up front: with clipping by the gradient's global norm or iRPROP+ the three calls simply run in turn. */
int myea_hip_backward_pass_update_derivative_weight_and_update_parameter(myea_hip_net *net, size_t batch_size, size_t training_size);

/* Neural_Network::Compute__Loss (Neural_Network__Compute__Loss__Loop.cpp:22-140, Neural_Network__Recurrent_Compute__Loss__Loop.cpp:20-140):
 * the evaluation twin of Compute__Error - the same loss and accuracy accumulation over the output layer's values, no
 * delta is written.  Used after a Forward_Pass in the inference state by Dataset::Testing (Dataset.cpp:7829-7860). */
int myea_hip_compute_loss(myea_hip_net *net, size_t batch_size_received, const float *desired_outputs, int desired_on_device);

/* Neural_Network::Compute__Accuracy__R (Neural_Network__Compute__R__Loop.cpp:22-90, Neural_Network__Recurrent_Compute__R__Loop.cpp):
 * second pass of the R accuracy.  The reference divides its two running sums by the number of entries in place
 * (Dataset::Measure_Accuracy, Dataset.cpp:7712-7713) and reads them back as the means; here the caller passes the
 * means (from myea_hip_get_loss) and the call adds to accuracy_r[1..3]. */
int myea_hip_compute_accuracy_r(myea_hip_net *net, size_t batch_size_received, const float *desired_outputs, int desired_on_device,
                                float desired_mean, float predicted_mean);

/* Device-side replacement of Dataset_Mini_Batch::Increment_Mini_Batch (Dataset__Mini_Batch.cpp:290-314), which
 * re-points an array of row pointers at the shuffled examples: copies rows `index[0..B)` of a dataset resident in
 * HBM ([examples][row_floats], fp32) into the contiguous batch `device_batch` ([B][row_floats]), ready to be
 * handed to forward_pass / compute_error / compute_loss with on_device = 1.  `index` is a host array, or a device
 * array when `index_on_device` != 0 (a whole epoch's permutation uploaded once).  No bound check on device
 * indices; host indices are checked against `dataset_examples`. */
int myea_hip_gather_examples(myea_hip_net *net, float *device_batch, const float *device_dataset, size_t dataset_examples,
                             size_t row_floats, const uint64_t *index, int index_on_device, size_t batch_size_received);

/* Device memory for a dataset kept in HBM (the reference's Dataset<T> keeps one host allocation per side and an array of
 * row pointers into it, Dataset.cpp `Allocate`; its CUDA twin copies both to the device, Dataset_Manager.cu).  `floats`
 * fp32 values, filled from `host` when that is not NULL.  The pointer is a plain device address: valid as `inputs` /
 * `desired_outputs` with on_device = 1 and as the source or destination of myea_hip_gather_examples. */
int myea_hip_device_buffer_create(size_t floats, const float *host, float **out_device);
int myea_hip_device_buffer_destroy(float *device);

/* Reset__Loss / the merged loss counters (Neural_Network__Merge.cpp:52-98).  get synchronises. */
int myea_hip_reset_loss(myea_hip_net *net);
int myea_hip_get_loss(myea_hip_net *net, myea_loss_state *out_state);

/* ---- debug taps (the reference's data members are public; these read the device copies) ---- */
int myea_hip_download_gradient(myea_hip_net *net, float *host_gradient, size_t count);
int myea_hip_upload_gradient(myea_hip_net *net, const float *host_gradient, size_t count);
int myea_hip_download_tensor(myea_hip_net *net, size_t layer_index, int kind, float *host, size_t count);
/* The running statistics of a normalised layer are network state that outlives a training run (the reference keeps them in
 * Normalized_unit::ptr_mean_average / ptr_variance_average and writes them into its dimension file, Neural_Network__Save.cpp:678-712).
 * `kind` = MYEA_TENSOR_NORM_MEANS_AVERAGES or MYEA_TENSOR_NORM_VARIANCES_AVERAGES, `count` = T x the layer's normalised units,
 * [T][units] as myea_hip_download_tensor returns them. */
int myea_hip_upload_tensor(myea_hip_net *net, size_t layer_index, int kind, const float *host, size_t count);

/* ---- profiling taps for the benchmark ---- */
/* When enabled, every dense-contraction (GEMM) launch is bracketed by HIP events on the net's stream;
 * myea_hip_profile_read() synchronises and returns accumulated launches / milliseconds / FLOPs per
 * family since the last reset.  family: 0 = forward (NT), 1 = dX (NN), 2 = dW (TN), 3 = optimizer
 * update (bytes instead of FLOPs), 4 = a layer's dX and dW contractions in one launch, 5 = the recurrent
 * contractions and gate math of an LSTM layer's forward time loop (steps 1 .. T-1; one launch per layer when the
 * loop runs as a resident kernel, one per step otherwise), 6 = the same of its backward time loop, 7 = batch
 * (re)normalisation forward and backward (bytes: every activation read or written once), 8 = column sums of the
 * deltas for the bias gradients (bytes), 9 = Compute__Error's output delta + loss kernel (bytes: outputs and desired values
 * read, delta written), 10 = the output layer's softmax (bytes: sums read, values written). */
int myea_hip_profile_enable(myea_hip_net *net, int enable);
int myea_hip_profile_read(myea_hip_net *net, int family, uint64_t *launches, double *milliseconds, double *work);

/* ---- kernel-level entry points on raw device pointers (stream = hipStream_t or NULL) ----
 * These are the kernels the net-level calls are built from, exported so that each one can be
 * checked and timed alone. */

/* C[M][N] (ldc) = (accumulate ? C : 0) + op(A) * op(B); fp32 MFMA.
 *   a_k_contiguous != 0: A is [M][K] with lda;  else A is [K][M] with lda.
 *   b_k_contiguous != 0: B is [N][K] with ldb;  else B is [K][N] with ldb.
 * Forward_Pass__FC (a=1,b=1), Backward_Pass__FC (a=1,b=0), Update_Derivative_Weight__FC (a=0,b=0). */
int myea_hip_gemm_f32(void *stream, int a_k_contiguous, int b_k_contiguous, int accumulate,
                      size_t M, size_t N, size_t K,
                      const float *A, size_t lda, const float *B, size_t ldb, float *C, size_t ldc);

/* Fused weight update over [0, count): Update_Parameters__{Adam,AMSGrad,AdaBound,AMSBound} and
 * Update_Parameter__Gradient_Descent{,_Momentum}, _Nesterov_Accelerated_Gradient, __iRPROP_plus, __iRPROP_minus.  `hyper`
 * supplies every scalar; optimizer_time_step is the value *after* the increment.  `gradient_scale` multiplies
 * the gradient on read (clip-by-norm fused; pass 1).  Unused state pointers may be NULL.
 * weight decay applies to indices < weight_count.
 * state0 / state1 / state2: gradient descent: previous deltas, -, -; the Adam family: first moment, second moment, its running
 * maximum (AMSGrad, AMSBound); iRPROP+: previous deltas, previous steps, previous derivatives (the step back is taken when
 * hyper->loss_rprop > hyper->previous_loss_rprop); iRPROP- (Neural_Network__iRPROP_minus.cpp:21-67): -, previous steps,
 * previous derivatives. */
int myea_hip_optimizer_update(void *stream, const myea_hyper *hyper, size_t count, size_t weight_count,
                              float gradient_scale, float *parameters, float *gradient,
                              float *state0, float *state1, float *state2);

/* ---- measured ceilings (no counterpart in the reference: figures for a benchmark's roofline) ----
 * myea_hip_ceiling_mfma_f32: a kernel of nothing but independent v_mfma_f32_32x32x2_f32, two wavefronts per SIMD,
 * `iterations` x 16 MFMAs per wavefront; best of `repeats` launches, in TFLOP/s.
 * myea_hip_ceiling_hbm_triad: a[i] = b[i] + s * c[i] over three arrays of `bytes_per_array` (allocated and freed by
 * the call; choose them well beyond the caches), one 16-byte element per lane and non-temporal stores as the optimizer
 * update has them; best of `repeats`, in GB/s of the 3 x bytes_per_array moved. */
int myea_hip_ceiling_mfma_f32(void *stream, int iterations, int repeats, double *tflops);
int myea_hip_ceiling_hbm_triad(void *stream, size_t bytes_per_array, int repeats, double *gigabytes_per_second);

#ifdef __cplusplus
}
#endif
#endif /* MYEA_HIP_H */
