// myea_net.h — the device-resident network object behind the C ABI (internal).
#pragma once

#include <hip/hip_runtime.h>

#include <utility>
#include <initializer_list>
#include <vector>

#include "../../include/myea_hip.h"
#include "myea_kernels.h"

namespace myea {

struct LstmLayer;  // myea_lstm.hip

struct DevLayer {
    size_t H = 0;  // *Layer::ptr_number_outputs
    // connections (Organize__Previous_Layers_Connected / Organize__Layer__Group, NN/Neural_Network.cpp:20-125)
    size_t prev = 0;  // previous_connected_layers[0]
    int group = 0;    // 0 outside a residual block, 1 first member of a block, 2 other members
    size_t In = 0;    // width of the producer
    // width of the activation-unit tensors (values, colscale) and of the normalised-unit tensors: H outside a block;
    // a block member carries both on its input side (In wide, no activation units on the first member); a residual
    // layer keeps its basic units in values / neuron_errors (H wide) and normalises the block's last member (NH wide)
    size_t AH = 0, NH = 0;
    size_t pad = 0;   // residual layer: column offset of the narrower shortcut operand (pooling_values[2])
    // [T][Bmax][H] (summations, neuron_errors), [T][Bmax][AH] (values), [T][Bmax][NH] (hats, normalizes)
    float *summations = nullptr, *values = nullptr, *hats = nullptr, *normalizes = nullptr, *neuron_errors = nullptr;
    float *in_errors = nullptr;  // normalised first member of a block: delta reduced to its input side [Bmax][In]
    // column sums of neuron_errors per block of 32 rows [ceil(T Bmax / 32)][H], left by the contraction that wrote the errors
    // (the bias gradient then sums the blocks instead of the rows); bias_partial_rows = blocks valid for a batch of
    // bias_partial_batch examples, 0 = the errors were written some other way
    float *bias_partials = nullptr;
    size_t bias_partial_rows = 0, bias_partial_batch = 0;
    // an independently recurrent layer: [Bmax][recurrent units], every example's share of the self weights' gradient (the sum over
    // the time steps of AF[t-1] dAF[t]), left by the backward time loop for du_rows_batch examples (0: not left in this pass)
    float *du_rows = nullptr;
    size_t du_rows_batch = 0;
    // a batch-normalised dense layer: [ceil(Bmax / 32)][2][H] column sums a contraction leaves for the normalisation's forward
    // (sum of x, of x * x) and backward pass (sum of dy * hats, of dy); consumed by the launch that follows it
    float *norm_partials = nullptr;
    // [T][NH]
    float *means = nullptr, *variances = nullptr, *means_averages = nullptr, *variances_averages = nullptr;
    float *r_corrections = nullptr, *d_corrections = nullptr;
    float *colscale = nullptr;  // dropout multiplier per (t, unit)
    unsigned long long colscale_epoch = 0;   // Net::mask_epoch the multipliers were derived at
    bool colscale_active = false;
    unsigned *pool_index = nullptr;  // max pooling: padded position each output took its value from [T][Bmax][H]
    // independently recurrent layer: pre-activations [T][Bmax][H]; the delta of the pre-activations lives in neuron_errors
    // unless a normalisation sits between the summation and the activation (then in dafs_own)
    float *pre_afs = nullptr, *dafs_own = nullptr;
    // Gaussian / Uout dropout: the draws of the forward pass [T][Bmax][H]; noise_uploaded: the caller's own, kept as they are
    float *noise = nullptr;
    bool noise_uploaded = false;
    int *unit_act = nullptr;    // per-unit activation types [AH], null = layer-wide
    float *unit_steep = nullptr;  // per-unit steepnesses [AH], null = layer-wide
    LstmLayer *lstm = nullptr, *lstm2 = nullptr;  // lstm2: the time-reversed direction of a bidirectional layer
};

constexpr int kProfFamilies = 11;   // forward, dX, dW, update, dX + dW launched as a pair, LSTM time loop forward, backward, normalisation, bias gradients, output error, softmax
constexpr int kProfLstmForwardLoop = 5, kProfLstmBackwardLoop = 6, kProfNormalization = 7, kProfBiasGradient = 8, kProfOutputError = 9, kProfSoftmax = 10;
struct ProfEvent {
    hipEvent_t start = nullptr, stop = nullptr;
    int family = 0;
    double work = 0;
    uint64_t launches = 1;   // launches between the two events (a recurrent layer's time loop is bracketed as a whole)
};

bool layer_is_pooling(const myea_layer_desc &l);
bool layer_is_ind_rnn(const myea_layer_desc &l);
bool layer_is_dense(const myea_layer_desc &l);
bool layer_uses_mask_dropout(const myea_layer_desc &l);
bool layer_uses_noise_dropout(const myea_layer_desc &l);
bool layer_uses_norm(const myea_layer_desc &l);
bool layer_uses_bias(const myea_layer_desc &l);

struct Net {
    myea_net_desc d{};
    myea_hyper h{};
    uint32_t state = MYEA_STATE_INFERENCE;
    hipStream_t stream = nullptr;
    // A stream of the library's own (default priority), forked from and joined to `stream` by events, for work that is
    // independent of what `stream` is busy with: the second direction of a bidirectional LSTM layer, and the bias /
    // peephole column reductions of the weight-gradient phase beside its contractions.
    hipStream_t side_stream = nullptr;
    hipEvent_t fork_event = nullptr, join_event = nullptr, update_event = nullptr;
    float *parameters = nullptr, *gradient = nullptr, *opt[MYEA_STATE_KINDS] = {};
    uint8_t *masks = nullptr;
    unsigned long long mask_epoch = 1;   // advances whenever the masks or the propagation state change
    unsigned long long dropout_seed = 0x9E3779B97F4A7C15ull, dropout_stream = 0;   // device generator: key and the next stream id
    uint8_t *zoneout_masks = nullptr;   // [state | output] halves, per LSTM layer [T][cells]
    size_t zoneout_count = 0;
    // max-norm constraint: weight segments (one per neuron / per LSTM gate vector), built on first use
    unsigned long long *seg_first = nullptr;
    unsigned *seg_len = nullptr;
    size_t n_segments = 0;
    unsigned longest_segment = 0;
    std::vector<DevLayer> L;
    float *tmp1 = nullptr, *tmp2 = nullptr, *scratch = nullptr, *stage_in = nullptr, *stage_out = nullptr;
    float *dw_slabs = nullptr;   // split-K slabs of a fully-connected weight gradient whose M x N is small and k long
    size_t scratch_floats = 0, dw_slab_floats = 0;   // sizes of the two buffers above
    // A sequence normalisation's backward launch leaves the scale's and the shift's gradient as shares per time step in the layer's
    // slice of bn_shares; ONE launch at the end of the backward pass adds the shares of every such layer onto the gradient
    // (flush_bn_shares).  bn_jobs: the table that launch reads, uploaded when the set of layers changes.
    float *bn_shares = nullptr;
    std::vector<size_t> bn_share_at;           // per layer: its slice's offset in floats, SIZE_MAX without one
    BnFoldJob *bn_jobs = nullptr, *bn_jobs_staging = nullptr;   // device; pinned host
    std::vector<BnFoldJob> bn_jobs_pending, bn_jobs_uploaded;
    int flush_bn_shares();
    // The same for the weight gradients of narrow layers (narrow_dw_slabs): a layer's slabs stay in its slice of narrow_slabs
    // until ONE launch at the end of Update_Derivative_Weight adds every layer's onto the gradient (flush_slab_folds).
    float *narrow_slabs = nullptr;
    size_t narrow_slab_floats = 0;
    std::vector<size_t> narrow_slab_at;        // per layer, SIZE_MAX without a slice
    SlabFoldJob *fold_jobs = nullptr, *fold_jobs_staging = nullptr;   // device; pinned host
    std::vector<SlabFoldJob> fold_pending, fold_uploaded;
    int flush_slab_folds();
    // the bounds of the independently recurrent layers' self weights, clipped behind every update in one launch; built at the first update
    ClipRange *clip_ranges = nullptr;
    size_t n_clip_ranges = 0, longest_clip_range = 0;
    bool clip_ranges_built = false;
    bool defer_folds = true;   // false: every layer's slabs are added right behind its contraction (a call that may not wait for the stream)
    float *static_scratch = nullptr;   // this device's copy of the library's static scratch array (update_derivative_weight_no_alloc)
    double *loss_acc = nullptr;                  // 8 doubles, see ErrorParams::loss_acc
    // LSTM time loops as one resident launch (myea_lstm_resident.hip): barrier counters in device memory, and a pinned host
    // word a kernel sets when one of its bounded waits gave up; resident_off: this network stays on one launch per time step
    unsigned *resident_sync = nullptr, *resident_flag = nullptr;
    // Bounded waits inside kernels (the time loops' barriers, the meeting of two workgroups that share a contraction's tile):
    // one that gives up raises resident_flag[0] (time loop) or resident_flag[1] (contraction) in pinned host memory and
    // `fault` in device memory.  While `fault` is set the update kernels change nothing, so no Update_Parameter enqueued behind
    // the incomplete pass steps the weights; the host word is reported by the next call that looks (resident_check()).
    unsigned *fault = nullptr;
    unsigned long long *updates_applied = nullptr;   // device counter: whole-vector updates that ran with `fault` clear
    // the optimizer's host-side scalars as they were before each update enqueued and not yet known to have run
    struct UpdateSnapshot { unsigned long long sequence; myea_hyper h; };
    std::vector<UpdateSnapshot> update_history;
    unsigned long long updates_enqueued = 0;
    bool gemm_pair_off = false;            // after a contraction's give-up: one workgroup per tile from then on
    void pair_buffers(GemmParams *g, float *partials, unsigned *tickets) const;   // a contraction's meeting place and fault words
    float *gemm_pair_partials = nullptr;       // scratch of the contractions that split a tile's k between two workgroups
    unsigned *gemm_pair_tickets = nullptr;
    float *resident_exchange = nullptr;   // partial sums the members of a group hand each other in the backward loop
    size_t resident_exchange_floats = 0;
    bool resident_off = false;
    int resident_check();   // MYEA_E_DEVICE (once) after a resident launch reported a give-up
    unsigned long long *index_stage = nullptr;   // [Bmax] example indices of a gathered batch

    bool profiling = false, open_event = false;
    std::vector<ProfEvent> pending, free_events;
    uint64_t prof_launches[kProfFamilies] = {};
    double prof_ms[kProfFamilies] = {}, prof_work[kProfFamilies] = {};

    ~Net();
    int create(const myea_net_desc &desc);
    int clear_optimizer();
    PoolParams pool_params(size_t li, size_t rows) const;
    int forward_pool_layer(size_t li, size_t B);
    int output_error_params(size_t B, const float *desired, int on_device, const char *fn, ErrorParams *p);
    int compute_loss(size_t B, const float *desired, int on_device);
    int compute_accuracy_r(size_t B, const float *desired, int on_device, float desired_mean, float predicted_mean);
    int gather_examples(float *dst, const float *src, size_t examples, size_t row_floats, const uint64_t *index, int index_on_device, size_t B);
    int build_max_norm_segments();
    float warm_restarts_decay(int *rc);

    float *layer_outputs(size_t li);
    float *scale_ptr(float *base, size_t li);
    float *shift_ptr(float *base, size_t li);
    void prof_begin(int family);
    void prof_end(double work, uint64_t launches = 1);
    void prof_cancel();

    int refresh_colscale(size_t li, bool *active);
    int forward_fc_layer(size_t li, size_t B);
    // act_out != nullptr (training only): the layer's activation and dropout multiplier ride in the normalisation's last pass
    // sums / sum_blocks: column sums the contraction that produced x (forward) or dy (backward) left per block of 32 rows
    int bn_forward(size_t li, size_t t, size_t rows, const float *x, bool training, float *act_out = nullptr, const float *colscale = nullptr,
                   const float *sums = nullptr, size_t sum_blocks = 0);
    int bn_backward(size_t li, size_t t, size_t rows, const float *x, const float *dy, float *dx, const float *sums = nullptr, size_t sum_blocks = 0);
    // the normalisation of layer li over all time steps of [T][batch_size][width] tensors
    int bn_forward_all(size_t li, size_t B, const float *x, bool training, float *act_out = nullptr, const float *colscale = nullptr);
    int bn_backward_all(size_t li, size_t B, const float *x, const float *dy, float *dx);
    int backward_into_layer(size_t li, size_t B);
    int pool_backward_with_shortcut(size_t gi, size_t rows, size_t roff, const DevLayer *shortcut, long crop, float *dst);
    int forward_residual_block(size_t ri, size_t B);
    int backward_residual_block(size_t ri, size_t B);

    int forward_pass(size_t B, const float *inputs, int on_device);
    int compute_error(size_t B, const float *desired, int on_device);
    int backward_pass(size_t B);
    // Backward_Pass followed by Update_Derivative_Weight over all layers, with a layer's weight gradient riding in the
    // launch that sends its delta down wherever the two contractions suit each other
    int backward_pass_and_update_derivative_weight(size_t B);
    bool pairing = false;              // inside the call above
    std::vector<char> dw_done;         // per layer: the weight contraction already ran in this pass
    // per layer: the layer's slice of the gradient is known to be zero (the update zeroes what it reads), so its next weight
    // contraction may store its product instead of adding it element by element at the L2.  MYEA_DW_STORE=0: always add.
    std::vector<char> dw_zero;
    void gradient_known_zero(bool zero) { dw_zero.assign(d.n_layers, zero ? 1 : 0); }
    bool dw_may_store(size_t li) const;
    bool fc_dw_params(size_t li, size_t B, GemmParams *g);   // false: the layer's weight gradient is not one plain contraction
    int update_derivative_weight(size_t B, size_t first, size_t end);
    int update_derivative_weight_contraction(size_t li, size_t B);   // the weight contraction(s) of one layer
    bool dw_beside_loop_allowed(size_t gi, size_t li, size_t B);
    bool dw_beside_loop = false;       // this pass put weight contractions on the side stream beside a time loop: join before returning
    bool loop_shares_device = false;   // set around a time loop that weight contractions will run beside
    // the same call with every scratch buffer of its kernels taken from the library's static device array
    int update_derivative_weight_no_alloc(size_t B, size_t first, size_t end);
    int update_parameter(size_t B, size_t training_size);
    // Update_Parameter in three parts: the step's scalars (advances the optimizer's time step), the elementwise update of a
    // range of the flat vectors, and what follows the update (constraints, repacking)
    int update_prepare(size_t B, size_t training_size, UpdateParams *p, double *bytes_per_param);
    int update_range(const UpdateParams &p, size_t first, size_t count, double bytes_per_param, bool last);   // last: the range that completes the update
    int update_finish();
    // Backward_Pass, Update_Derivative_Weight over all layers and Update_Parameter as one call: the weights of a
    // fully-connected layer take their step on the side stream as soon as their gradient is complete and nothing reads them
    // any more in this pass, beside the contractions of the layers below
    int backward_pass_update_derivative_weight_and_update_parameter(size_t B, size_t training_size);
    bool early_update_allowed() const;
    int early_update_layer(size_t li);
    const UpdateParams *early_update = nullptr;              // inside the call above, when it updates early
    double early_bytes_per_param = 0;
    std::vector<std::pair<size_t, size_t>> early_ranges;     // [first, end) of the flat vectors updated so far in this call
    int set_unit_activations(size_t li, const uint32_t *types, const float *steep, size_t count);

    // LSTM-with-peephole layers (myea_lstm.hip)
    int lstm_create_layer(size_t li);
    void lstm_destroy_layer(DevLayer &o);
    int lstm_parameters_changed();
    int lstm_pair_words_clear();   // the meeting words of the LSTM layers' shared-tile contractions back to zero
    int lstm_forward_layer(size_t li, size_t B);
    int lstm_backward_layer(size_t li, size_t B);       // BPTT inside LSTM layer li
    // delta / weight operands an LSTM consumer gi offers to the layer below: delta [T][Bmax][width], weights [width][fan-in]
    void lstm_delta_source(size_t gi, int direction, const float **delta, size_t *width, const float **weights);
    bool lstm_backward_loop_leaves_room(size_t li, size_t B);   // the layer's resident backward loop occupies at most half of the compute units
    int side_stream_create();
    int side_stream_join();            // `stream` waits for what the last SideStreamScope enqueued
    int lstm_forward_inputs(size_t li, LstmLayer &q, size_t B);
    int lstm_forward_step(LstmLayer &q, size_t B, size_t s);
    int lstm_resident_dirs(DevLayer &o, LstmResidentDir *dirs);   // the layer's directions as the resident kernels take them
    int lstm_backward_step(LstmLayer &q, size_t B, size_t s);
    // a normalised layer's time steps, and the normalisation of a list of its nine groups of normalised units at one step
    int lstm_forward_step_norm(LstmLayer &q, size_t B, size_t s);
    int lstm_backward_step_norm(LstmLayer &q, size_t B, size_t s);
    int lstm_norm_forward_groups(LstmLayer &q, size_t B, size_t t, std::initializer_list<int> groups);
    int lstm_norm_backward_groups(LstmLayer &q, size_t B, size_t t, std::initializer_list<int> groups);
    float *lstm_norm_statistics(size_t li, int kind, size_t *count);   // running averages of one group (kind carries the group)
    int lstm_update_derivative_weight_direction(size_t li, LstmLayer &q, size_t B);
    size_t lstm_scratch_floats() const;
    // packed weight-gradient slabs of all LSTM directions: their total size (each rounded up to 64 floats), and
    // re-pointing them into `base` (null: back to the layers' own buffers)
    size_t lstm_gradient_slab_floats() const;
    void lstm_bind_gradient_slabs(float *base);
    int lstm_update_derivative_weight(size_t li, size_t B, bool reductions);
    int lstm_update_derivative_weight_reductions(LstmLayer &q, size_t B);
    const float *lstm_tensor(size_t li, int kind, size_t *count);
};

// Launches made while the scope lives go to the side stream, ordered behind everything `stream` held when it opened.
struct SideStreamScope {
    Net &net;
    bool active = false;
    explicit SideStreamScope(Net &n) : net(n)
    {
        if (!n.side_stream || hipEventRecord(n.fork_event, n.stream) != hipSuccess || hipStreamWaitEvent(n.side_stream, n.fork_event, 0) != hipSuccess) return;
        std::swap(n.stream, n.side_stream);
        active = true;
    }
    ~SideStreamScope()
    {
        if (!active) return;
        std::swap(net.stream, net.side_stream);
        (void)hipEventRecord(net.join_event, net.side_stream);
    }
    SideStreamScope(const SideStreamScope &) = delete;
    SideStreamScope &operator=(const SideStreamScope &) = delete;
};

}  // namespace myea
