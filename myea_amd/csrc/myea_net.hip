// myea_net.hip — the device-resident network behind the C ABI: buffers, the five step entry points and
// the movement of parameters / optimizer state.  Host code only; the kernels live in myea_gemm.hip and
// myea_elementwise.hip (and myea_lstm.hip).
//
// NN/ = Neural_Network_Library_Windows/Source_Files/Neural_Network/ of the reference.
#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "myea_kernels.h"
#include "myea_net.h"

namespace myea {

// ---- error plumbing ---------------------------------------------------------------------------------
static thread_local char g_last_error[512] = "";

void set_last_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
}

int hip_fail(hipError_t e, const char *what)
{
    set_last_error("HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
    return MYEA_E_DEVICE;
}

// ---- static device scratch ------------------------------------------------------------------------------
// Scratch memory of the allocation-free entry point (myea_hip_update_derivative_weight_no_alloc): partial sums of the
// column reductions and split-K slabs live here instead of in buffers the library allocates.  Every device the
// library runs on holds its own copy of the array, at its own address, until the process ends; in host code the
// array's name is only a handle for hipGetSymbolAddress, never a device address.
constexpr size_t kStaticScratchFloats = (size_t)8 << 20;   // 32 MiB
static __device__ __align__(256) float static_scratch[kStaticScratchFloats];

constexpr int kMaxDevices = 64;
static float *g_static_scratch_address[kMaxDevices] = {};
static std::mutex g_static_scratch_mutex;

// the current device's copy of the array; resolved once per device
static int static_scratch_address(float **out)
{
    int dev = -1;
    MYEA_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) { set_last_error("static scratch: device ordinal %d out of range", dev); return MYEA_E_DEVICE; }
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (!g_static_scratch_address[dev]) {
        void *p = nullptr;
        MYEA_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch)));
        if (!p) { set_last_error("static scratch: hipGetSymbolAddress returned a null address"); return MYEA_E_DEVICE; }
        g_static_scratch_address[dev] = static_cast<float *>(p);
    }
    *out = g_static_scratch_address[dev];
    return MYEA_OK;
}

// ---- small helpers ------------------------------------------------------------------------------------
static int dev_alloc(float **p, size_t count)
{
    *p = nullptr;
    void *q = nullptr;
    hipError_t e = hipMalloc(&q, (count ? count : 1) * sizeof(float));
    if (e != hipSuccess) { hip_fail(e, "hipMalloc"); return MYEA_E_NOMEM; }
    *p = static_cast<float *>(q);
    return MYEA_OK;
}

#define MYEA_TRY(expr)                 \
    do {                               \
        int rc__ = (expr);             \
        if (rc__ != MYEA_OK) return rc__; \
    } while (0)

bool layer_is_pooling(const myea_layer_desc &l) { return l.type_layer == MYEA_LAYER_AVERAGE_POOLING || l.type_layer == MYEA_LAYER_MAX_POOLING; }
bool layer_is_ind_rnn(const myea_layer_desc &l) { return l.type_layer == MYEA_LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT; }
// layers made of neuron units and activation units
bool layer_is_dense(const myea_layer_desc &l) { return l.type_layer == MYEA_LAYER_FULLY_CONNECTED || layer_is_ind_rnn(l); }
bool layer_uses_mask_dropout(const myea_layer_desc &l) { return l.type_dropout == MYEA_DROPOUT_BERNOULLI || l.type_dropout == MYEA_DROPOUT_BERNOULLI_INVERTED; }
bool layer_uses_noise_dropout(const myea_layer_desc &l) { return l.type_dropout == MYEA_DROPOUT_GAUSSIAN || l.type_dropout == MYEA_DROPOUT_UOUT; }
bool layer_uses_norm(const myea_layer_desc &l) { return l.type_normalization != MYEA_NORMALIZATION_NONE; }
bool layer_uses_bias(const myea_layer_desc &l) { return !layer_uses_norm(l); }  // Layer::Use__Bias, Data.hpp:736

float *Net::layer_outputs(size_t li)
{
    const myea_layer_desc &l = d.layers[li];
    DevLayer &o = L[li];
    if (li != 0 && layer_is_dense(l)) {
        if (o.group) return o.summations;  // residual group: the member's output is its summation (NN/Neural_Network__Ordered.cpp:96-141)
        if (layer_uses_norm(l) && !l.use_layer_normalization_before_activation) return o.normalizes;
    }
    return o.values;  // LSTM: cell outputs; residual layer: its basic units' values
}

float *Net::scale_ptr(float *base, size_t li) { return base + d.total_weights + d.total_bias + d.layers[li].first_normalized_unit_index; }
float *Net::shift_ptr(float *base, size_t li) { return scale_ptr(base, li) + d.total_normalized_units; }

// ---- profiling ------------------------------------------------------------------------------------------
void Net::prof_begin(int family)
{
    if (!profiling) return;
    ProfEvent ev;
    ev.family = family;
    if (!free_events.empty()) { ev = free_events.back(); free_events.pop_back(); ev.family = family; }
    else if (hipEventCreate(&ev.start) != hipSuccess || hipEventCreate(&ev.stop) != hipSuccess) return;
    (void)hipEventRecord(ev.start, stream);
    pending.push_back(ev);
    open_event = true;
}

// drops the pair opened by prof_begin when nothing was launched after all
void Net::prof_cancel()
{
    if (!profiling || !open_event) return;
    free_events.push_back(pending.back());
    pending.pop_back();
    open_event = false;
}

void Net::prof_end(double work, uint64_t launches)
{
    if (!profiling || !open_event) return;
    ProfEvent &ev = pending.back();
    ev.work = work;
    ev.launches = launches;
    (void)hipEventRecord(ev.stop, stream);
    open_event = false;
}

static int check_desc(const myea_net_desc &d)
{
    if (d.n_layers < 2 || d.n_layers > MYEA_MAX_LAYERS) { set_last_error("descriptor: %u layers (need 2..%d)", d.n_layers, MYEA_MAX_LAYERS); return MYEA_E_INVALID; }
    if (d.batch_size == 0 || d.number_recurrent_depth == 0) { set_last_error("descriptor: batch_size and number_recurrent_depth must be >= 1"); return MYEA_E_INVALID; }
    if (d.total_parameters != d.total_weights + d.total_bias + 2 * d.total_normalized_units) { set_last_error("descriptor: total_parameters inconsistent"); return MYEA_E_INVALID; }
    if (d.layers[0].type_layer != MYEA_LAYER_FULLY_CONNECTED) { set_last_error("descriptor: the input layer must be a fully-connected (unit) layer"); return MYEA_E_INVALID; }
    // residual blocks: members are the block_depth layers after the residual layer, a consumer follows.  group: 0 outside a
    // block, 1 a dense first member, 2 another dense member, 3 a pooling member, 4 an LSTM member
    bool any_lstm = false;
    uint32_t block_end = 0;  // index of the last member of the block being walked, 0 outside
    std::vector<int> group(d.n_layers, 0);
    for (uint32_t li = 0; li < d.n_layers; ++li) {
        const myea_layer_desc &l = d.layers[li];
        if (!layer_is_dense(l) && l.type_layer != MYEA_LAYER_LSTM && l.type_layer != MYEA_LAYER_RESIDUAL && !layer_is_pooling(l)) {
            set_last_error("layer %u: type %u is not on this path", li, l.type_layer);
            return MYEA_E_UNSUPPORTED;
        }
        if (block_end != 0) {
            if (l.type_layer == MYEA_LAYER_RESIDUAL) { set_last_error("layer %u: a residual block inside a residual block is not on this path", li); return MYEA_E_UNSUPPORTED; }
            group[li] = layer_is_pooling(l) ? 3 : (l.type_layer == MYEA_LAYER_LSTM ? 4 : ((d.layers[li - 1].type_layer == MYEA_LAYER_RESIDUAL) ? 1 : 2));
            if (li == block_end) block_end = 0;
        } else if (l.type_layer == MYEA_LAYER_RESIDUAL) {
            if (l.block_depth == 0 || (uint64_t)li + l.block_depth + 1 >= d.n_layers) { set_last_error("layer %u: residual block of depth %u does not fit in front of a consumer", li, l.block_depth); return MYEA_E_INVALID; }
            if (l.type_dropout != MYEA_DROPOUT_NONE && l.type_dropout != MYEA_DROPOUT_SHAKEDROP) { set_last_error("layer %u: a residual layer's dropout is ShakeDrop or none", li); return MYEA_E_UNSUPPORTED; }
            if (l.type_dropout == MYEA_DROPOUT_SHAKEDROP && !(l.dropout_values[0] >= 0.f && l.dropout_values[0] <= 1.f)) { set_last_error("layer %u: ShakeDrop probability %g", li, (double)l.dropout_values[0]); return MYEA_E_INVALID; }
            block_end = li + l.block_depth;
        }
        if (l.type_layer == MYEA_LAYER_LSTM) any_lstm = true;
    }
    (void)any_lstm;
    for (uint32_t li = 0; li < d.n_layers; ++li) {
        const myea_layer_desc &l = d.layers[li];
        if (l.k_sparsity != 0) {
            // hidden fully-connected layers; inside a residual block on the member's input-side activation units (none on a first member)
            const float scaled = (float)l.k_sparsity * l.alpha_sparsity;
            const size_t width = group[li] == 2 ? (size_t)myea_net_desc_number_outputs(&d, myea_net_desc_previous_layer(&d, li)) : l.n_units;
            if (li == 0 || li + 1 >= d.n_layers || l.type_layer != MYEA_LAYER_FULLY_CONNECTED || group[li] == 1) { set_last_error("layer %u: the k-sparse filter is on this path for hidden fully-connected layers that own activation units", li); return MYEA_E_UNSUPPORTED; }
            if (l.k_sparsity > width || !(l.alpha_sparsity >= 0.f) || !(scaled >= 1.f) || (uint64_t)scaled > width) { set_last_error("layer %u: k-sparse filter: k %u, alpha %g do not fit %zu units", li, l.k_sparsity, (double)l.alpha_sparsity, width); return MYEA_E_INVALID; }
        }
        if (layer_is_ind_rnn(l)) {
            if (li == 0 || li + 1 >= d.n_layers) { set_last_error("layer %u: an independently recurrent layer is a hidden layer", li); return MYEA_E_INVALID; }
            if (l.type_activation_function == MYEA_AF_SOFTMAX) { set_last_error("layer %u: softmax belongs to the output layer only", li); return MYEA_E_UNSUPPORTED; }
            if (l.constraint_recurrent_weight_lower_bound > l.constraint_recurrent_weight_upper_bound) { set_last_error("layer %u: recurrent weight bounds out of order", li); return MYEA_E_INVALID; }
            // inside a block the recurrence sits on the member's input side, fan-in wide; the reference's backward pass walks it with
            // the member's output width (NN/Neural_Network__Backward_Pass__OpenMP.cpp:867-877), which only addresses it when the two are equal
            if (group[li] == 2 && myea_net_desc_number_outputs(&d, myea_net_desc_previous_layer(&d, li)) != l.n_units) {
                set_last_error("layer %u: an independently recurrent member of a residual block is as wide as its input on this path (as in the reference's own indexing)", li);
                return MYEA_E_UNSUPPORTED;
            }
        }
        if (layer_is_pooling(l)) {
            // the width must be the one Assign__Post__Layer computes (NN/Neural_Network__Compile.cpp:250-271) - the kernels index with it
            if (li == 0 || li + 1 >= d.n_layers) { set_last_error("layer %u: a pooling layer sits between the input and the output layer", li); return MYEA_E_UNSUPPORTED; }
            const double in = (double)myea_net_desc_number_outputs(&d, myea_net_desc_previous_layer(&d, li)), k = l.pooling_values[0], st = l.pooling_values[1], pad = l.pooling_values[2], dil = l.pooling_values[3];
            if (k < 1 || st < 1) { set_last_error("layer %u: pooling kernel and stride must be >= 1", li); return MYEA_E_INVALID; }
            const double span = l.type_layer == MYEA_LAYER_AVERAGE_POOLING ? in + 2 * pad - k : in + 2 * pad - dil * (k - 1) - 1;
            const double out = span < 0 ? 0 : (l.pooling_values[4] == 0 ? std::floor(span / st + 1.0) : std::ceil(span / st + 1.0));
            if (out < 1 || (double)l.n_units != out) { set_last_error("layer %u: pooling width %u does not follow from its parameters (%.0f)", li, l.n_units, out); return MYEA_E_INVALID; }
            // (a normalisation type on a pooling layer is accepted and means nothing: the reference's setter takes any hidden layer,
            // NN/Neural_Network__Layer_Normalization.cpp:217-288, the layer owns no normalised unit and its passes never look at the field)
            if (l.type_dropout != MYEA_DROPOUT_NONE) { set_last_error("layer %u: a pooling layer carries no dropout", li); return MYEA_E_UNSUPPORTED; }
        }
    }
    for (uint32_t li = 0; li < d.n_layers; ++li) {
        const myea_layer_desc &l = d.layers[li];
        if (l.type_layer == MYEA_LAYER_RESIDUAL) {
            const uint64_t nh = myea_net_desc_number_outputs(&d, li + l.block_depth);
            if (layer_uses_norm(l) && l.first_normalized_unit_index + nh > d.total_normalized_units) { set_last_error("layer %u: scale/shift slice leaves its region", li); return MYEA_E_INVALID; }
            if (l.type_normalization > MYEA_NORMALIZATION_BATCH_RENORMALIZATION) { set_last_error("layer %u: normalization type %u is not on this path", li, l.type_normalization); return MYEA_E_UNSUPPORTED; }
            continue;
        }
        if (l.n_units == 0) { set_last_error("layer %u: no units", li); return MYEA_E_INVALID; }
        if (layer_is_pooling(l)) continue;
        if (l.type_dropout == MYEA_DROPOUT_ZONEOUT && l.type_layer == MYEA_LAYER_LSTM) {
            // masks per (time step, cell), uploaded with myea_hip_upload_zoneout_masks
        } else if (layer_uses_noise_dropout(l)) {
            // one draw per (time step, example, activation unit): hidden / output fully-connected layers; a block's first member owns no such unit
            if (li == 0 || l.type_layer != MYEA_LAYER_FULLY_CONNECTED || group[li] == 1) { set_last_error("layer %u: Gaussian / Uout dropout is on this path for fully-connected layers that own activation units", li); return MYEA_E_UNSUPPORTED; }
            if (!(l.dropout_values[0] >= 0.f)) { set_last_error("layer %u: dropout value %g", li, (double)l.dropout_values[0]); return MYEA_E_INVALID; }
        } else if (l.type_dropout != MYEA_DROPOUT_NONE && !layer_uses_mask_dropout(l)) {
            set_last_error("layer %u: dropout type %u is not on this path", li, l.type_dropout);
            return MYEA_E_UNSUPPORTED;
        }
        if (l.type_normalization > MYEA_NORMALIZATION_BATCH_RENORMALIZATION) { set_last_error("layer %u: normalization type %u is not on this path", li, l.type_normalization); return MYEA_E_UNSUPPORTED; }
        if (layer_is_dense(l) && li > 0) {
            const bool has_af = group[li] != 1;
            if (has_af && (l.type_activation_function == MYEA_AF_NONE || l.type_activation_function >= MYEA_AF_LENGTH)) { set_last_error("layer %u: activation %u invalid", li, l.type_activation_function); return MYEA_E_INVALID; }
            if (group[li] == 2 && l.type_activation_function == MYEA_AF_SOFTMAX) { set_last_error("layer %u: softmax belongs to the output layer only", li); return MYEA_E_UNSUPPORTED; }
            const size_t fan_in = (size_t)myea_net_desc_number_outputs(&d, myea_net_desc_previous_layer(&d, li));
            const size_t units_af = group[li] == 0 ? l.n_units : (group[li] == 1 ? 0 : fan_in), units_norm = group[li] == 0 ? l.n_units : fan_in;
            if (l.first_connection_index + fan_in * l.n_units + (layer_is_ind_rnn(l) ? units_af : 0u) > d.total_weights) { set_last_error("layer %u: weight slice leaves the weight region", li); return MYEA_E_INVALID; }
            if (layer_uses_bias(l) && l.first_bias_connection_index + l.n_units > d.total_weights + d.total_bias) { set_last_error("layer %u: bias slice leaves the bias region", li); return MYEA_E_INVALID; }
            if (layer_uses_norm(l) && l.first_normalized_unit_index + units_norm > d.total_normalized_units) { set_last_error("layer %u: scale/shift slice leaves its region", li); return MYEA_E_INVALID; }
            if (l.type_dropout != MYEA_DROPOUT_NONE && l.first_mask_index + (uint64_t)units_af * d.number_recurrent_depth > d.total_mask_units) { set_last_error("layer %u: mask slice leaves the mask buffer", li); return MYEA_E_INVALID; }
            if (l.type_dropout != MYEA_DROPOUT_NONE && group[li] == 1) { set_last_error("layer %u: the first layer of a residual block has no activation unit to drop", li); return MYEA_E_INVALID; }
        }
        if (li == 0 && l.type_dropout != MYEA_DROPOUT_NONE &&
            l.first_mask_index + (uint64_t)l.n_units * d.number_recurrent_depth > d.total_mask_units) { set_last_error("layer %u: mask slice leaves the mask buffer", li); return MYEA_E_INVALID; }
    }
    return MYEA_OK;
}

static int fc_dw_slabs(size_t H, size_t In, size_t rows, size_t first_connection_index);

int Net::create(const myea_net_desc &desc)
{
    MYEA_TRY(check_desc(desc));
    d = desc;
    for (uint32_t li = 0; li < d.n_layers; ++li)   // see check_desc: the field means nothing on a pooling layer
        if (layer_is_pooling(d.layers[li])) d.layers[li].type_normalization = MYEA_NORMALIZATION_NONE;
    myea_hyper_default(&h);
    const size_t P = d.total_parameters, T = d.number_recurrent_depth, B = d.batch_size;
    MYEA_TRY(dev_alloc(&parameters, P));
    MYEA_TRY(dev_alloc(&gradient, P));
    for (int k = 0; k < MYEA_STATE_KINDS; ++k) MYEA_TRY(dev_alloc(&opt[k], P));
    MYEA_HIP_TRY(hipMemset(parameters, 0, P * sizeof(float)));
    MYEA_HIP_TRY(hipMemset(gradient, 0, P * sizeof(float)));
    gradient_known_zero(true);
    for (int k = 0; k < MYEA_STATE_KINDS; ++k) MYEA_HIP_TRY(hipMemset(opt[k], 0, P * sizeof(float)));
    MYEA_TRY(launch_fill(0, opt[MYEA_STATE_PREVIOUS_STEPS], P, h.rprop_delta_zero));
    if (d.total_normalized_units) MYEA_TRY(launch_fill(0, parameters + d.total_weights + d.total_bias, d.total_normalized_units, 1.f));
    {
        void *q = nullptr;
        MYEA_HIP_TRY(hipMalloc(&q, d.total_mask_units ? d.total_mask_units : 1));
        masks = static_cast<uint8_t *>(q);
        MYEA_HIP_TRY(hipMemset(masks, 1, d.total_mask_units ? d.total_mask_units : 1));  // all true, NN/Neural_Network__Allocate.cpp:386-410
        size_t cells = 0;
        for (size_t li = 1; li < d.n_layers; ++li)
            if (d.layers[li].type_layer == MYEA_LAYER_LSTM) cells += (size_t)d.layers[li].n_units * d.layers[li].n_cells_per_block * (d.layers[li].use_bidirectional ? 2 : 1);
        zoneout_count = 2 * T * cells;
        MYEA_HIP_TRY(hipMalloc(&q, zoneout_count ? zoneout_count : 1));
        zoneout_masks = static_cast<uint8_t *>(q);
        MYEA_HIP_TRY(hipMemset(zoneout_masks, 1, zoneout_count ? zoneout_count : 1));  // all true, NN/Neural_Network__Allocate.cpp:1209-1211
    }
    size_t max_h = 0;
    L.resize(d.n_layers);
    for (size_t li = 0; li < d.n_layers; ++li) {
        const myea_layer_desc &l = d.layers[li];
        DevLayer &o = L[li];
        o.H = (size_t)myea_net_desc_number_outputs(&d, (uint32_t)li);
        o.prev = myea_net_desc_previous_layer(&d, (uint32_t)li);
        o.In = li ? (size_t)myea_net_desc_number_outputs(&d, (uint32_t)o.prev) : 0;
        o.group = 0;
        {   // inside a residual block: the layer right behind a residual layer, and every layer up to the block's depth
            bool member = false;
            for (size_t r = 1; r < li && !member; ++r) member = d.layers[r].type_layer == MYEA_LAYER_RESIDUAL && li <= r + d.layers[r].block_depth;
            if (member) {
                if (layer_is_dense(l)) o.group = d.layers[li - 1].type_layer == MYEA_LAYER_RESIDUAL ? 1 : 2;
                else if (layer_is_pooling(l)) o.group = 3;   // basic units as wide as the layer, no activation or normalised units
                else if (l.type_layer == MYEA_LAYER_LSTM) o.group = 4;   // the layer as it is outside a block
            }
        }
        if (l.type_layer == MYEA_LAYER_RESIDUAL) {
            o.NH = (size_t)myea_net_desc_number_outputs(&d, (uint32_t)(li + l.block_depth));
            o.AH = o.H;
            o.pad = ((o.In > o.NH ? o.In - o.NH : o.NH - o.In) + 1) / 2;  // Assign__Post__Layer, NN/Neural_Network__Compile.cpp:277
        } else {
            const bool own_width = o.group == 0 || o.group >= 3;
            o.AH = own_width ? o.H : (o.group == 1 ? 0 : o.In);
            o.NH = own_width ? o.H : o.In;
        }
        if (o.H > max_h) max_h = o.H;
        const size_t sz = T * B * o.H, sa = T * B * o.AH, sn = T * B * o.NH;
        MYEA_TRY(dev_alloc(&o.values, sa));
        MYEA_HIP_TRY(hipMemset(o.values, 0, (sa ? sa : 1) * sizeof(float)));
        if (layer_uses_mask_dropout(l) && layer_is_dense(l)) MYEA_TRY(dev_alloc(&o.colscale, T * o.AH));
        if (l.type_layer == MYEA_LAYER_RESIDUAL && l.type_dropout == MYEA_DROPOUT_SHAKEDROP) {   // [T][B] masks, [T][B][NH] forward draws, [T][B][NH] backward draws
            MYEA_TRY(dev_alloc(&o.noise, T * (B + 2 * B * o.NH)));
            MYEA_HIP_TRY(hipMemset(o.noise, 0, T * (B + 2 * B * o.NH) * sizeof(float)));
        }
        if (layer_uses_noise_dropout(l)) {   // one draw per activation unit
            MYEA_TRY(dev_alloc(&o.noise, sa));
            MYEA_TRY(launch_fill(0, o.noise, sa, l.type_dropout == MYEA_DROPOUT_GAUSSIAN ? 1.f : 0.f));   // neutral until a pass draws
        }
        if (li == 0) continue;
        if (l.type_layer == MYEA_LAYER_LSTM) { MYEA_TRY(lstm_create_layer(li)); continue; }
        if (l.type_layer == MYEA_LAYER_MAX_POOLING) {
            void *q = nullptr;
            MYEA_HIP_TRY(hipMalloc(&q, (sz ? sz : 1) * sizeof(unsigned)));
            o.pool_index = static_cast<unsigned *>(q);
            MYEA_HIP_TRY(hipMemset(o.pool_index, 0, (sz ? sz : 1) * sizeof(unsigned)));
        }
        if (l.type_layer != MYEA_LAYER_RESIDUAL && !layer_is_pooling(l)) {
            MYEA_TRY(dev_alloc(&o.summations, sz));
            MYEA_HIP_TRY(hipMemset(o.summations, 0, sz * sizeof(float)));
        }
        MYEA_TRY(dev_alloc(&o.neuron_errors, sz));  // residual layer: its basic units' errors
        if (layer_is_dense(l) && layer_uses_bias(l) && li + 1 < d.n_layers) MYEA_TRY(dev_alloc(&o.bias_partials, (T * B + 31) / 32 * o.H));
        if (layer_is_dense(l) && l.type_normalization == MYEA_NORMALIZATION_BATCH_NORMALIZATION) MYEA_TRY(dev_alloc(&o.norm_partials, (B + 31) / 32 * 2 * (o.H > o.NH ? o.H : o.NH)));
        MYEA_HIP_TRY(hipMemset(o.neuron_errors, 0, sz * sizeof(float)));
        if (layer_is_ind_rnn(l) && o.group != 1) {   // a block's first member owns no recurrent unit: a plain member
            const size_t su = o.group ? sa : sz;     // inside a block the recurrent units sit on the input side
            MYEA_TRY(dev_alloc(&o.pre_afs, su));
            MYEA_HIP_TRY(hipMemset(o.pre_afs, 0, su * sizeof(float)));
            if (T > 1) MYEA_TRY(dev_alloc(&o.du_rows, su / T));   // [Bmax][recurrent units]
            // the delta of the pre-activations IS the neuron errors unless a normalisation sits between the two; a block member
            // always keeps its own (what it hands to the member before it may be changed by that member afterwards)
            if (o.group || (layer_uses_norm(l) && l.use_layer_normalization_before_activation)) {
                MYEA_TRY(dev_alloc(&o.dafs_own, su));
                MYEA_HIP_TRY(hipMemset(o.dafs_own, 0, su * sizeof(float)));
            }
        }
        if (layer_uses_norm(l)) {
            MYEA_TRY(dev_alloc(&o.hats, sn));
            MYEA_TRY(dev_alloc(&o.normalizes, sn));
            MYEA_HIP_TRY(hipMemset(o.hats, 0, sn * sizeof(float)));
            MYEA_HIP_TRY(hipMemset(o.normalizes, 0, sn * sizeof(float)));
            if (o.group == 1) {
                MYEA_TRY(dev_alloc(&o.in_errors, sn));
                MYEA_HIP_TRY(hipMemset(o.in_errors, 0, sn * sizeof(float)));
            }
            float **small[] = {&o.means, &o.variances, &o.means_averages, &o.variances_averages, &o.r_corrections, &o.d_corrections};
            for (float **s : small) { MYEA_TRY(dev_alloc(s, T * o.NH)); MYEA_HIP_TRY(hipMemset(*s, 0, T * o.NH * sizeof(float))); }
            MYEA_TRY(launch_fill(0, o.variances_averages, T * o.NH, 1.f));  // NN/Neural_Network__Allocate.cpp:2612-2615
        }
    }
    MYEA_TRY(side_stream_create());
    {   // forward contractions of few tiles split each tile's k between two workgroups: their meeting place
        MYEA_TRY(dev_alloc(&gemm_pair_partials, (size_t)kGemmPairTiles * 128 * 128));
        void *q = nullptr;
        MYEA_HIP_TRY(hipMalloc(&q, 2 * kGemmPairTiles * sizeof(unsigned)));
        MYEA_HIP_TRY(hipMemset(q, 0, 2 * kGemmPairTiles * sizeof(unsigned)));
        gemm_pair_tickets = static_cast<unsigned *>(q);
        // what a kernel's bounded wait raises when it gives up: a device word the update kernels look at (behind it, 8 bytes on,
        // the count of updates that ran) and two pinned host words the next call that looks reports
        MYEA_HIP_TRY(hipMalloc(&q, 16));
        MYEA_HIP_TRY(hipMemset(q, 0, 16));
        fault = static_cast<unsigned *>(q);
        updates_applied = reinterpret_cast<unsigned long long *>(fault + 2);
        MYEA_HIP_TRY(hipHostMalloc(&q, 64, hipHostMallocDefault));
        resident_flag = static_cast<unsigned *>(q);
        resident_flag[0] = resident_flag[1] = 0u;
    }
    {
        bool any_lstm = false;
        for (size_t li = 1; li < d.n_layers; ++li) any_lstm = any_lstm || d.layers[li].type_layer == MYEA_LAYER_LSTM;
        if (any_lstm) {   // counters and flags of the resident time loops
            void *q = nullptr;
            MYEA_HIP_TRY(hipMalloc(&q, lstm_resident_sync_words() * sizeof(unsigned)));
            resident_sync = static_cast<unsigned *>(q);
            if (resident_exchange_floats) MYEA_TRY(dev_alloc(&resident_exchange, resident_exchange_floats));
        }
    }
    MYEA_TRY(dev_alloc(&tmp1, T * B * max_h));
    MYEA_TRY(dev_alloc(&tmp2, T * B * max_h));
    bn_share_at.assign(d.n_layers, SIZE_MAX);
    if (T > 1) {   // a slice per normalised dense layer or block for the per-time-step shares of its scale / shift gradient
        size_t need = 0, count = 0;
        for (size_t li = 1; li < d.n_layers; ++li)
            if (layer_uses_norm(d.layers[li]) && d.layers[li].type_layer != MYEA_LAYER_LSTM && L[li].NH) { bn_share_at[li] = need; need += (2 * T * L[li].NH + 63) / 64 * 64; ++count; }
        if (count) {
            MYEA_TRY(dev_alloc(&bn_shares, need));
            void *q = nullptr;
            MYEA_HIP_TRY(hipMalloc(&q, count * sizeof(BnFoldJob)));
            bn_jobs = static_cast<BnFoldJob *>(q);
            MYEA_HIP_TRY(hipHostMalloc(&q, count * sizeof(BnFoldJob), hipHostMallocDefault));
            bn_jobs_staging = static_cast<BnFoldJob *>(q);
        }
    }
    {
        size_t need = 258 * max_h + 2048;
        if (2 * T * max_h > need) need = 2 * T * max_h;   // a sequence's normalisation: the scale / shift gradient shares per time step
        if (lstm_scratch_floats() > need) need = lstm_scratch_floats();
        MYEA_TRY(dev_alloc(&scratch, need));
        scratch_floats = need;
    }
    {   // weight gradients of narrow layers over long T x batch row ranges run as split-K contractions into slabs
        size_t need = 0;
        for (size_t li = 1; li < d.n_layers; ++li) {
            if (!layer_is_dense(d.layers[li])) continue;
            const int slabs = fc_dw_slabs(L[li].H, L[li].In, T * B, d.layers[li].first_connection_index);
            if (slabs > 1) need = std::max(need, (size_t)slabs * L[li].H * L[li].In);
        }
        if (need) MYEA_TRY(dev_alloc(&dw_slabs, need));
        dw_slab_floats = need;
        // the narrow ones among them keep their slabs until the end of the call: a slice each
        narrow_slab_at.assign(d.n_layers, SIZE_MAX);
        size_t pool = 0, count = 0;
        for (size_t li = 1; li < d.n_layers; ++li) {
            if (!layer_is_dense(d.layers[li])) continue;
            const int slabs = narrow_dw_slabs(L[li].H, L[li].In, T * B);
            if (slabs > 0) { narrow_slab_at[li] = pool; pool += ((size_t)slabs * L[li].H * L[li].In + 63) / 64 * 64; ++count; }
            if (L[li].du_rows) ++count;   // the shares of an independently recurrent layer's self weights go through the same table
        }
        narrow_slab_floats = pool;
        if (count) {
            if (pool) MYEA_TRY(dev_alloc(&narrow_slabs, pool));
            void *q = nullptr;
            MYEA_HIP_TRY(hipMalloc(&q, count * sizeof(SlabFoldJob)));
            fold_jobs = static_cast<SlabFoldJob *>(q);
            MYEA_HIP_TRY(hipHostMalloc(&q, count * sizeof(SlabFoldJob), hipHostMallocDefault));
            fold_jobs_staging = static_cast<SlabFoldJob *>(q);
        }
    }
    MYEA_TRY(static_scratch_address(&static_scratch));   // set-up: this device's address of the static array
    MYEA_TRY(dev_alloc(&stage_in, T * B * L[0].H));
    MYEA_TRY(dev_alloc(&stage_out, T * B * L[d.n_layers - 1].H));
    {
        void *q = nullptr;
        MYEA_HIP_TRY(hipMalloc(&q, 8 * sizeof(double)));
        loss_acc = static_cast<double *>(q);
        MYEA_HIP_TRY(hipMemset(loss_acc, 0, 8 * sizeof(double)));
        MYEA_HIP_TRY(hipMalloc(&q, B * sizeof(unsigned long long)));
        index_stage = static_cast<unsigned long long *>(q);
    }
    MYEA_HIP_TRY(hipDeviceSynchronize());
    return MYEA_OK;
}

Net::~Net()
{
    if (side_stream) {
        (void)hipStreamSynchronize(side_stream);
        (void)hipStreamDestroy(side_stream);
        (void)hipEventDestroy(fork_event);
        (void)hipEventDestroy(join_event);
        if (update_event) (void)hipEventDestroy(update_event);
    }
    auto fr = [](void *p) { if (p) (void)hipFree(p); };
    fr(parameters); fr(gradient);
    for (int k = 0; k < MYEA_STATE_KINDS; ++k) fr(opt[k]);
    fr(seg_first); fr(seg_len);
    fr(masks); fr(zoneout_masks);
    for (DevLayer &o : L) {
        fr(o.summations); fr(o.values); fr(o.hats); fr(o.normalizes); fr(o.neuron_errors); fr(o.in_errors); fr(o.bias_partials); fr(o.norm_partials); fr(o.colscale); fr(o.unit_act); fr(o.unit_steep); fr(o.pool_index); fr(o.pre_afs); fr(o.dafs_own); fr(o.du_rows); fr(o.noise);
        fr(o.means); fr(o.variances); fr(o.means_averages); fr(o.variances_averages); fr(o.r_corrections); fr(o.d_corrections);
        lstm_destroy_layer(o);
    }
    fr(resident_sync);
    fr(resident_exchange);
    fr(gemm_pair_partials); fr(gemm_pair_tickets); fr(fault);
    if (resident_flag) (void)hipHostFree(resident_flag);
    fr(bn_shares); fr(bn_jobs); fr(narrow_slabs); fr(fold_jobs); fr(clip_ranges);
    if (fold_jobs_staging) (void)hipHostFree(fold_jobs_staging);
    if (bn_jobs_staging) (void)hipHostFree(bn_jobs_staging);
    fr(tmp1); fr(tmp2); fr(scratch); fr(stage_in); fr(stage_out); fr(loss_acc); fr(index_stage); fr(dw_slabs);
    for (ProfEvent &e : pending) { (void)hipEventDestroy(e.start); (void)hipEventDestroy(e.stop); }
    for (ProfEvent &e : free_events) { (void)hipEventDestroy(e.start); (void)hipEventDestroy(e.stop); }
}

// ---- dropout column multipliers ---------------------------------------------------------------------------
// Training: Bernoulli -> mask ? 1 : 0; inverted -> mask ? 1/keep : 0 (NN/Neural_Network__Forward_Pass__OpenMP.cpp:
// 628-647, 4907-4966).  Inference: Bernoulli scales by keep (:4968-4990); inverted does nothing.
int Net::refresh_colscale(size_t li, bool *active)
{
    const myea_layer_desc &l = d.layers[li];
    DevLayer &o = L[li];
    *active = false;
    if (!layer_uses_mask_dropout(l) || !o.colscale) return MYEA_OK;
    if (o.colscale_epoch == mask_epoch) { *active = o.colscale_active; return MYEA_OK; }   // same masks, same state: still valid
    const size_t n = (size_t)d.number_recurrent_depth * o.AH;
    if (state == MYEA_STATE_TRAINING) {
        float on = 1.f;
        if (l.type_dropout == MYEA_DROPOUT_BERNOULLI_INVERTED) on = l.dropout_values[0] == 0.f ? 0.f : 1.f / l.dropout_values[0];
        MYEA_TRY(launch_mask_to_scale(stream, n, masks + l.first_mask_index, on, o.colscale));
        *active = true;
    } else if (l.type_dropout == MYEA_DROPOUT_BERNOULLI) {
        MYEA_TRY(launch_fill(stream, o.colscale, n, l.dropout_values[0]));
        *active = true;
    }
    o.colscale_epoch = mask_epoch;
    o.colscale_active = *active;
    return MYEA_OK;
}

// ---- forward ----------------------------------------------------------------------------------------------
// Forward_Pass__FC (layer driver), NN/Neural_Network__Forward_Pass__OpenMP.cpp:256-698:
// GEMM -> bias -> [BN before] -> activation / softmax -> [BN after] -> dropout.
// MYEA_BN_SUMS_FROM_GEMM=0 in the environment keeps the normalisation's column sums in kernels of their own, =f / =b takes them
// from the contraction in the forward / backward pass only (for A / B runs)
static bool bn_sums_from_gemm(bool backward = false)
{
    static const int mode = [] { const char *e = std::getenv("MYEA_BN_SUMS_FROM_GEMM"); return !e || !*e ? 3 : e[0] == '0' ? 0 : e[0] == 'f' ? 1 : e[0] == 'b' ? 2 : 3; }();
    return (mode & (backward ? 2 : 1)) != 0;
}

// The normalisation of every time step of a [T][Bmax][width] tensor: one launch for the whole sequence (each time step keeps
// statistics of its own); MYEA_BN_SEQUENCE=0 in the environment keeps one set of launches per time step (for A / B runs).
static bool bn_sequence_allowed()
{
    static const bool on = [] { const char *e = std::getenv("MYEA_BN_SEQUENCE"); return !(e && e[0] == '0'); }();
    return on;
}

int Net::forward_fc_layer(size_t li, size_t B)
{
    const myea_layer_desc &l = d.layers[li];
    DevLayer &o = L[li];
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size, In = o.In, H = o.H;
    const float *x = layer_outputs(o.prev);
    const bool norm = layer_uses_norm(l), before = l.use_layer_normalization_before_activation != 0;
    const bool softmax = l.type_activation_function == MYEA_AF_SOFTMAX;
    const bool training = state >= MYEA_STATE_TRAINING;
    const bool ind = layer_is_ind_rnn(l);
    bool drop = false;
    MYEA_TRY(refresh_colscale(li, &drop));
    // all time steps in one launch when the rows are contiguous and nothing is per time step; a normalisation in front of the
    // activation has its own statistics per time step inside one launch (with the activation and the dropout multiplier of each)
    const bool af_in_bn_ok = training && !ind && !softmax && !o.unit_act;
    const bool seq_bn = T > 1 && norm && before && B == Bmax && bn_sequence_allowed() && 2 * T * H <= scratch_floats && (ind || !drop || af_in_bn_ok);
    const bool per_t = T > 1 && !seq_bn && (B != Bmax || norm || (drop && !ind));
    const size_t chunks = per_t ? T : 1, rows = per_t ? B : (T > 1 ? T * B : B);
    for (size_t c = 0; c < chunks; ++c) {
        const size_t roff = c * Bmax;  // first row of the chunk
        const float *cs = drop ? o.colscale + c * H : nullptr;
        GemmParams g{};
        g.A = x + roff * In; g.lda = (long)In; g.a_k_contiguous = 1;
        g.B = parameters + l.first_connection_index; g.ldb = (long)In; g.b_k_contiguous = 1;
        g.C = o.summations + roff * H; g.ldc = (long)H;
        g.M = (int)rows; g.N = (int)H; g.K = (int)In;
        g.epilogue = EPI_FC_FORWARD;
        g.bias = layer_uses_bias(l) ? parameters + l.first_bias_connection_index : nullptr;
        g.act = (int)l.type_activation_function;
        const bool fuse_af = !ind && !softmax && !(norm && before) && !o.unit_act && gemm_can_fuse_activation((int)l.type_activation_function);
        g.aux_out = fuse_af ? o.values + roff * H : nullptr;
        g.colscale = (fuse_af && !norm) ? cs : nullptr;
        // a batch normalisation in front of the activation, training: its column sums leave with the contraction's tiles
        const bool sums_from_gemm = !seq_bn && norm && before && training && o.norm_partials && bn_sums_from_gemm() && l.type_normalization == MYEA_NORMALIZATION_BATCH_NORMALIZATION && o.NH == H;
        if (sums_from_gemm) g.col_partials = o.norm_partials;
        pair_buffers(&g, gemm_pair_partials, gemm_pair_tickets);   // forward contractions run one at a time on this stream
        prof_begin(0);
        MYEA_TRY(launch_gemm(stream, g));
        prof_end(2.0 * (double)rows * (double)H * (double)In);

        const float *cur = o.summations + roff * H;
        // training: the activation of a layer normalised first rides in the normalisation's last pass
        const bool af_in_bn = norm && before && training && !ind && !softmax && !o.unit_act;
        if (norm && before) {
            if (seq_bn) MYEA_TRY(bn_forward_all(li, B, cur, training, af_in_bn ? o.values : nullptr, cs));
            else MYEA_TRY(bn_forward(li, c, rows, cur, training, af_in_bn ? o.values + roff * H : nullptr, cs, sums_from_gemm ? o.norm_partials : nullptr, (rows + 31) / 32));
            cur = o.normalizes + roff * H;
        }
        if (ind) continue;   // the recurrence and the activation follow for the whole sequence
        if (softmax) {
            prof_begin(kProfSoftmax);
            MYEA_TRY(launch_softmax(stream, rows, H, cur, o.values + roff * H, norm ? nullptr : cs));
            prof_end((double)rows * (double)H * sizeof(float) * 2.0);   // sums read once, values written once
        }
        else if (!fuse_af && !af_in_bn) MYEA_TRY(launch_activation(stream, (int)l.type_activation_function, rows, H, cur, o.values + roff * H, cs, o.unit_act));
        if (norm && !before) {
            MYEA_TRY(bn_forward(li, c, rows, o.values + roff * H, training));
            if (cs) MYEA_TRY(launch_colscale(stream, rows, H, o.normalizes + roff * H, cs));
        }
        // Gaussian / Uout dropout on the layer's outputs, strictly in the training state (:716-750)
        if (o.noise && state == MYEA_STATE_TRAINING) {
            if (c == 0 && !o.noise_uploaded) {   // fresh draws for the whole sequence, one stream id per (pass, layer)
                const bool normal = l.type_dropout == MYEA_DROPOUT_GAUSSIAN;
                MYEA_TRY(launch_dropout_noise(stream, T * Bmax * H, o.noise, normal ? 1 : 0, normal ? 1.f : -l.dropout_values[0], l.dropout_values[0], dropout_seed, dropout_stream++));
            }
            MYEA_TRY(launch_dropout_noise_apply(stream, rows * H, ((norm && !before) ? o.normalizes : o.values) + roff * H, o.noise + roff * H, l.type_dropout == MYEA_DROPOUT_UOUT));
        }
        // k-Sparse, after the dropout (NN/Neural_Network__Forward_Pass__Loop.cpp:752-790): k values stay strictly in the
        // training state, size_t(alpha k) otherwise
        if (l.k_sparsity != 0) {
            const size_t k = state == MYEA_STATE_TRAINING ? (size_t)l.k_sparsity : (size_t)(l.alpha_sparsity * (float)l.k_sparsity);
            MYEA_TRY(launch_k_sparse(stream, rows, H, k, ((norm && !before) ? o.normalizes : o.values) + roff * H));
        }
    }
    if (ind) {
        // Forward_Pass__FC_Ind_RNN + Forward_Pass__FC_AF (NN/Neural_Network__Forward_Pass__Loop.cpp:434-470): the dropout of an
        // un-normalised layer works in place on the activations the next time step reads, so it rides in the same kernel
        const bool after = norm && !before;
        IndRnnParams p{};
        p.T = T; p.B = B; p.Bmax = Bmax; p.H = H;
        p.u = parameters + l.first_connection_index + H * In;
        p.act = (int)l.type_activation_function; p.unit_act = o.unit_act;
        p.in = (norm && before) ? o.normalizes : o.summations;
        p.pre_afs = o.pre_afs; p.afs = o.values;
        p.colscale = (drop && !after) ? o.colscale : nullptr;
        MYEA_TRY(launch_ind_rnn_forward(stream, p));
        if (after) {
            for (size_t t = 0; t < T; ++t) {
                MYEA_TRY(bn_forward(li, t, B, o.values + t * Bmax * H, training));
                if (drop) MYEA_TRY(launch_colscale(stream, B, H, o.normalizes + t * Bmax * H, o.colscale + t * H));
            }
        }
    }
    return MYEA_OK;
}

int Net::bn_forward(size_t li, size_t t, size_t rows, const float *x, bool training, float *act_out, const float *colscale, const float *sums, size_t sum_blocks)
{
    const myea_layer_desc &l = d.layers[li];
    DevLayer &o = L[li];
    const size_t H = o.NH, roff = t * d.batch_size;
    if (!training) {
        return launch_bn_forward_inference(stream, rows, H, x, scale_ptr(parameters, li), shift_ptr(parameters, li),
                                           o.means_averages + t * H, o.variances_averages + t * H, o.normalizes + roff * H);
    }
    BnForwardParams p{};
    p.rows = rows; p.H = H; p.x = x;
    p.scale = scale_ptr(parameters, li); p.shift = shift_ptr(parameters, li);
    p.mean = o.means + t * H; p.var = o.variances + t * H;
    p.mean_avg = o.means_averages + t * H; p.var_avg = o.variances_averages + t * H;
    p.r_corr = o.r_corrections + t * H; p.d_corr = o.d_corrections + t * H;
    p.hats = o.hats + roff * H; p.normalizes = o.normalizes + roff * H;
    p.epsilon = h.normalization_epsilon; p.momentum = h.normalization_momentum_average;
    p.r_max = h.batch_renormalization_r_correction_maximum; p.d_max = h.batch_renormalization_d_correction_maximum;
    p.renorm = l.type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
    p.act_out = act_out; p.colscale = colscale; p.act = (int)l.type_activation_function;
    // algorithmic bytes: x read once, the normalised values (x-hat) and the scaled and shifted output written once
    prof_begin(kProfNormalization);
    const int rc = (sums && !p.renorm) ? launch_bn_forward_training_from_sums(stream, p, sums, sum_blocks) : launch_bn_forward_training(stream, p, scratch);
    prof_end((double)rows * (double)H * sizeof(float) * (act_out ? 4.0 : 3.0));
    return rc;
}

int Net::bn_forward_all(size_t li, size_t B, const float *x, bool training, float *act_out, const float *colscale)
{
    const myea_layer_desc &l = d.layers[li];
    DevLayer &o = L[li];
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size, H = o.NH;
    if (T == 1 || !bn_sequence_allowed() || 2 * T * H > scratch_floats) {
        for (size_t t = 0; t < T; ++t)
            MYEA_TRY(bn_forward(li, t, B, x + t * Bmax * H, training, act_out ? act_out + t * Bmax * H : nullptr, colscale ? colscale + t * H : nullptr));
        return MYEA_OK;
    }
    BnForwardParams p{};
    p.rows = B; p.H = H; p.x = x;
    p.scale = scale_ptr(parameters, li); p.shift = shift_ptr(parameters, li);
    p.mean = o.means; p.var = o.variances; p.mean_avg = o.means_averages; p.var_avg = o.variances_averages;
    p.r_corr = o.r_corrections; p.d_corr = o.d_corrections;
    p.hats = o.hats; p.normalizes = o.normalizes;
    p.epsilon = h.normalization_epsilon; p.momentum = h.normalization_momentum_average;
    p.r_max = h.batch_renormalization_r_correction_maximum; p.d_max = h.batch_renormalization_d_correction_maximum;
    p.renorm = l.type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
    p.act_out = act_out; p.colscale = colscale; p.act = (int)l.type_activation_function;
    prof_begin(kProfNormalization);
    const int rc = launch_bn_forward_sequence(stream, p, T, Bmax, training ? 1 : 0);
    prof_end((double)T * (double)B * (double)H * sizeof(float) * (training ? (act_out ? 4.0 : 3.0) : 2.0));
    return rc;
}

int Net::bn_backward_all(size_t li, size_t B, const float *x, const float *dy, float *dx)
{
    const myea_layer_desc &l = d.layers[li];
    DevLayer &o = L[li];
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size, H = o.NH;
    if (T == 1 || !bn_sequence_allowed() || 2 * T * H > scratch_floats || bn_share_at[li] == SIZE_MAX) {
        for (size_t t = T; t-- > 0;) MYEA_TRY(bn_backward(li, t, B, x + t * Bmax * H, dy + t * Bmax * H, dx + t * Bmax * H));
        return MYEA_OK;
    }
    BnBackwardParams p{};
    p.rows = B; p.H = H; p.x = x; p.hats = o.hats; p.dy = dy;
    p.mean = o.means; p.var = o.variances; p.scale = scale_ptr(parameters, li); p.r_corr = o.r_corrections;
    p.dscale = scale_ptr(gradient, li); p.dshift = shift_ptr(gradient, li);
    p.dx = dx;
    p.renorm = l.type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
    prof_begin(kProfNormalization);
    // the shares of the scale's and the shift's gradient stay in the layer's slice until the end of the pass: flush_bn_shares
    float *shares = bn_shares + bn_share_at[li];
    const int rc = launch_bn_backward_sequence(stream, p, T, Bmax, shares, false);
    prof_end((double)T * (double)B * (double)H * sizeof(float) * 3.0);
    if (rc == MYEA_OK) bn_jobs_pending.push_back(BnFoldJob{shares, p.dscale, p.dshift, (unsigned)H, (unsigned)T});
    return rc;
}

// The slabs the narrow layers' weight gradients of this call left are added onto the gradient: one launch for all layers.
int Net::flush_slab_folds()
{
    if (fold_pending.empty()) return MYEA_OK;
    const size_t count = fold_pending.size();
    bool same = fold_uploaded.size() == count;
    for (size_t i = 0; same && i < count; ++i) same = std::memcmp(&fold_pending[i], &fold_uploaded[i], sizeof(SlabFoldJob)) == 0;
    if (!same) {   // the first call, or one over other layers or buffers than the last: the table goes up again
        MYEA_HIP_TRY(hipStreamSynchronize(stream));   // no earlier launch still reads the table
        std::memcpy(fold_jobs_staging, fold_pending.data(), count * sizeof(SlabFoldJob));
        MYEA_HIP_TRY(hipMemcpyAsync(fold_jobs, fold_jobs_staging, count * sizeof(SlabFoldJob), hipMemcpyHostToDevice, stream));
        MYEA_HIP_TRY(hipStreamSynchronize(stream));   // the staging words are free again
        fold_uploaded = fold_pending;
    }
    size_t widest = 0;
    for (const SlabFoldJob &j : fold_pending) widest = std::max(widest, (size_t)j.n);
    fold_pending.clear();
    prof_begin(2);
    const int rc = launch_slab_fold_jobs(stream, fold_jobs, count, widest);
    prof_end(0.0);
    return rc;
}

// The shares every sequence normalisation of this backward pass left are added onto the gradient: one launch for all layers.
int Net::flush_bn_shares()
{
    if (bn_jobs_pending.empty()) return MYEA_OK;
    const size_t count = bn_jobs_pending.size();
    bool same = bn_jobs_uploaded.size() == count;
    for (size_t i = 0; same && i < count; ++i) same = std::memcmp(&bn_jobs_pending[i], &bn_jobs_uploaded[i], sizeof(BnFoldJob)) == 0;
    if (!same) {   // the first pass, or one over other layers than the last (another batch size): the table goes up again
        MYEA_HIP_TRY(hipStreamSynchronize(stream));   // no earlier launch still reads the table
        std::memcpy(bn_jobs_staging, bn_jobs_pending.data(), count * sizeof(BnFoldJob));
        MYEA_HIP_TRY(hipMemcpyAsync(bn_jobs, bn_jobs_staging, count * sizeof(BnFoldJob), hipMemcpyHostToDevice, stream));
        MYEA_HIP_TRY(hipStreamSynchronize(stream));   // the staging words are free again
        bn_jobs_uploaded = bn_jobs_pending;
    }
    size_t widest = 0;
    for (const BnFoldJob &j : bn_jobs_pending) widest = std::max(widest, (size_t)j.H);
    bn_jobs_pending.clear();
    prof_begin(kProfNormalization);
    const int rc = launch_bn_share_folds(stream, bn_jobs, count, widest);
    prof_end(0.0);
    return rc;
}

// A kernel whose bounded wait gave up - a resident LSTM time loop, or a contraction whose tiles two workgroups share - has left
// the pass it belonged to incomplete.  From that kernel on the device-side fault word is set and every update kernel behind
// it has changed nothing.  The next call that looks reports it, once: everything enqueued runs to its end, the host-side
// optimizer scalars go back to what they were before the first update that did not run, the gradient is cleared, the fault
// words and the contractions' meeting words are reset, and the network keeps to the plain forms (one launch per time step,
// one workgroup per tile) from then on.  The caller repeats the mini-batch.
int Net::resident_check()
{
    if (!resident_flag || (resident_flag[0] == 0u && resident_flag[1] == 0u)) return MYEA_OK;
    MYEA_HIP_TRY(hipStreamSynchronize(stream));
    if (side_stream) MYEA_HIP_TRY(hipStreamSynchronize(side_stream));
    const unsigned loop_code = resident_flag[0], pair_code = resident_flag[1];
    resident_flag[0] = resident_flag[1] = 0u;
    if (loop_code) resident_off = true;
    if (pair_code) gemm_pair_off = true;
    unsigned long long applied = 0;
    MYEA_HIP_TRY(hipMemcpy(&applied, updates_applied, sizeof(applied), hipMemcpyDeviceToHost));
    bool rolled_back = applied == updates_enqueued;
    for (const UpdateSnapshot &snap : update_history) {
        if (snap.sequence != applied) continue;
        // the scalars an update advances (update_prepare, warm_restarts_decay, clear_optimizer); what the caller set stays
        h.optimizer_time_step = snap.h.optimizer_time_step; h.adam_previous_beta2 = snap.h.adam_previous_beta2;
        h.epoch_time_step = snap.h.epoch_time_step; h.warm_restarts_T_i = snap.h.warm_restarts_T_i;
        h.warm_restarts_maximum_learning_rate = snap.h.warm_restarts_maximum_learning_rate;
        h.loss_rprop = snap.h.loss_rprop; h.previous_loss_rprop = snap.h.previous_loss_rprop;
        rolled_back = true;
        break;
    }
    const unsigned long long skipped = updates_enqueued - applied;
    updates_enqueued = applied;
    update_history.clear();
    MYEA_HIP_TRY(hipMemset(fault, 0, sizeof(unsigned)));
    MYEA_HIP_TRY(hipMemset(gemm_pair_tickets, 0, 2 * kGemmPairTiles * sizeof(unsigned)));
    MYEA_HIP_TRY(hipMemset(gradient, 0, d.total_parameters * sizeof(float)));
    gradient_known_zero(true);
    MYEA_TRY(lstm_pair_words_clear());
    const char *what = loop_code == 2u ? "resident LSTM time loop: the workgroups of a group did not share an XCD"
                       : loop_code    ? "resident LSTM time loop: a wait between time steps gave up (workgroups not resident together?)"
                                      : "contraction with tiles shared by two workgroups: the wait for a tile's other half gave up";
    set_last_error("%s; the pass is incomplete, %llu update(s) enqueued behind it changed nothing%s, the gradient is cleared; later passes use %s",
                   what, skipped, rolled_back ? "" : " (the optimizer's time step could not be taken back)",
                   loop_code ? "one launch per time step" : "one workgroup per tile");
    return MYEA_E_DEVICE;
}

void Net::pair_buffers(GemmParams *g, float *partials, unsigned *tickets) const
{
    if (gemm_pair_off) return;
    g->pair_partials = partials; g->pair_tickets = tickets;
    g->pair_fault = fault; g->pair_host_flag = resident_flag ? resident_flag + 1 : nullptr;
    g->pair_polls = gemm_pair_polls();
}

// FF__Forward_Pass_Batch (NN/Neural_Network__Forward_Pass__OpenMP.cpp:24-120) / RNN__Forward_Pass_Batch
// (NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:24-130): assign inputs, then layer by layer.
int Net::forward_pass(size_t B, const float *inputs, int on_device)
{
    MYEA_TRY(resident_check());
    if (!inputs) { set_last_error("Forward_Pass: null inputs"); return MYEA_E_INVALID; }
    if (B == 0 || B > d.batch_size) { set_last_error("Forward_Pass: batch size (%zu) > maximum batch size (%u)", B, d.batch_size); return MYEA_E_BATCH; }
    const size_t T = d.number_recurrent_depth, In = L[0].H, Bmax = d.batch_size;
    const size_t n = B * T * In;
    if (T == 1) {
        MYEA_HIP_TRY(hipMemcpyAsync(L[0].values, inputs, n * sizeof(float), on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, stream));
    } else {
        const float *src = inputs;
        if (!on_device) {
            MYEA_HIP_TRY(hipMemcpyAsync(stage_in, inputs, n * sizeof(float), hipMemcpyHostToDevice, stream));
            src = stage_in;
        }
        MYEA_TRY(launch_scatter_time_major(stream, B, T, In, Bmax, src, L[0].values));
    }
    bool drop = false;
    MYEA_TRY(refresh_colscale(0, &drop));
    if (drop) {
        for (size_t t = 0; t < T; ++t) MYEA_TRY(launch_colscale(stream, B, In, L[0].values + t * Bmax * In, L[0].colscale + t * In));
    }
    for (size_t li = 1; li < d.n_layers; ++li) {
        if (layer_is_dense(d.layers[li])) MYEA_TRY(forward_fc_layer(li, B));
        else if (layer_is_pooling(d.layers[li])) MYEA_TRY(forward_pool_layer(li, B));
        else if (d.layers[li].type_layer == MYEA_LAYER_RESIDUAL) {
            MYEA_TRY(forward_residual_block(li, B));
            li += d.layers[li].block_depth;  // the walk resumes after the block's last member
        } else MYEA_TRY(lstm_forward_layer(li, B));
    }
    return MYEA_OK;
}

PoolParams Net::pool_params(size_t li, size_t rows) const
{
    const myea_layer_desc &l = d.layers[li];
    PoolParams p{};
    p.rows = rows; p.In = L[li].In; p.H = L[li].H;
    p.kernel = l.pooling_values[0]; p.stride = l.pooling_values[1]; p.padding = l.pooling_values[2]; p.dilation = l.pooling_values[3];
    p.is_max = l.type_layer == MYEA_LAYER_MAX_POOLING;
    return p;
}

int Net::forward_pool_layer(size_t li, size_t B)
{
    DevLayer &o = L[li];
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size;
    const float *x = layer_outputs(o.prev);
    const bool per_t = T > 1 && B != Bmax;
    const size_t chunks = per_t ? T : 1, rows = per_t ? B : T * B;
    for (size_t c = 0; c < chunks; ++c) {
        const size_t roff = c * Bmax;
        MYEA_TRY(launch_pool_forward(stream, pool_params(li, rows), x + roff * o.In, o.values + roff * o.H, o.pool_index ? o.pool_index + roff * o.H : nullptr));
    }
    return MYEA_OK;
}

// Forward_Pass__Residual (NN/Neural_Network__Forward_Pass__OpenMP.cpp:3861-3997) over pre-activation members
// (Forward_Pass__Residual__FC, :4039-4433): on the member's INPUT [BN] -> (not the first member: [+ u * AF[t-1]] -> activation ->
// dropout -> k-sparse filter), then weights and bias; the member's output is its summation.  The activation (+ Bernoulli
// dropout) of member m+1 is applied by the epilogue of member m's contraction whenever nothing else sits between them.
// After the last member: [block-level BN], [ShakeDrop], then the zero-padded identity shortcut (:5158-5240).
// With a recurrent depth the members run one after the other, each over all of its time steps
// (Recurrent__Forward_Pass__Residual / __Residual__Layer, NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:563-771): a
// dense or pooling member time step by time step (every normalisation has its own statistics per time step), an
// independently recurrent member's recurrence and an LSTM member's time loop as the layers of that kind outside a block.
int Net::forward_residual_block(size_t ri, size_t B)
{
    const myea_layer_desc &r = d.layers[ri];
    const size_t last = ri + r.block_depth, T = d.number_recurrent_depth, Bmax = d.batch_size;
    const bool training = state >= MYEA_STATE_TRAINING;
    // Launches that treat every row alike cover the whole sequence when the batch fills the network's rows (the time steps are
    // then contiguous); one per time step otherwise, or when something differs from one time step to the next (by_step)
    auto chunked = [&](bool by_step, auto &&launch) -> int {
        const bool split = T > 1 && (by_step || B != Bmax);
        const size_t n = split ? T : 1, rows = split ? B : T * B;
        for (size_t c = 0; c < n; ++c) MYEA_TRY(launch(c, c * Bmax, rows));
        return MYEA_OK;
    };
    bool values_ready = false;  // the member's activation values were written by the previous member's contractions
    for (size_t m = ri + 1; m <= last; ++m) {
        const myea_layer_desc &l = d.layers[m];
        DevLayer &o = L[m];
        const size_t In = o.In, H = o.H;
        const float *x = layer_outputs(o.prev);
        if (l.type_layer == MYEA_LAYER_LSTM) {
            MYEA_TRY(lstm_forward_layer(m, B));
            values_ready = false;
            continue;
        }
        if (layer_is_pooling(l)) {   // a pooling member (Forward_Pass__Residual__Layer, :4005-4030): windows over the member before it
            MYEA_TRY(chunked(false, [&](size_t, size_t roff, size_t rows) {
                return launch_pool_forward(stream, pool_params(m, rows), x + roff * In, o.values + roff * H, o.pool_index ? o.pool_index + roff * H : nullptr);
            }));
            values_ready = false;
            continue;
        }
        bool drop = false;
        if (o.group == 2) MYEA_TRY(refresh_colscale(m, &drop));
        const bool norm = layer_uses_norm(l), ind = o.group == 2 && layer_is_ind_rnn(l);
        if (norm) MYEA_TRY(bn_forward_all(m, B, x, training));
        const float *in = norm ? o.normalizes : x;
        if (ind) {   // the recurrence and the activation over the whole sequence; Bernoulli dropout in place on what the next step reads
            IndRnnParams p{};
            p.T = T; p.B = B; p.Bmax = Bmax; p.H = In;
            p.u = parameters + l.first_connection_index + H * In;
            p.act = (int)l.type_activation_function; p.unit_act = o.unit_act;
            p.in = in; p.pre_afs = o.pre_afs; p.afs = o.values;
            p.colscale = drop ? o.colscale : nullptr;
            MYEA_TRY(launch_ind_rnn_forward(stream, p));
        }
        if (o.group == 2) {
            if (!ind && !values_ready)
                MYEA_TRY(chunked(drop, [&](size_t t, size_t roff, size_t rows) {
                    return launch_activation(stream, (int)l.type_activation_function, rows, In, in + roff * In, o.values + roff * In, drop ? o.colscale + t * o.AH : nullptr, o.unit_act);
                }));
            // Gaussian / Uout dropout, strictly in the training state, then the k-sparse filter (:4197-4274)
            if (o.noise && state == MYEA_STATE_TRAINING) {
                if (!o.noise_uploaded) {
                    const bool normal = l.type_dropout == MYEA_DROPOUT_GAUSSIAN;
                    MYEA_TRY(launch_dropout_noise(stream, T * Bmax * In, o.noise, normal ? 1 : 0, normal ? 1.f : -l.dropout_values[0], l.dropout_values[0], dropout_seed, dropout_stream++));
                }
                MYEA_TRY(chunked(false, [&](size_t, size_t roff, size_t rows) {
                    return launch_dropout_noise_apply(stream, rows * In, o.values + roff * In, o.noise + roff * In, l.type_dropout == MYEA_DROPOUT_UOUT);
                }));
            }
            if (l.k_sparsity != 0) {
                const size_t k = state == MYEA_STATE_TRAINING ? (size_t)l.k_sparsity : (size_t)(l.alpha_sparsity * (float)l.k_sparsity);
                MYEA_TRY(chunked(false, [&](size_t, size_t roff, size_t rows) { return launch_k_sparse(stream, rows, In, k, o.values + roff * In); }));
            }
            in = o.values;
        }
        // what the contractions of this member leave for the next one: its activation values, when only an activation and a
        // Bernoulli multiplier stand between the two
        bool feeds_next = false;
        if (m < last) {
            const myea_layer_desc &nx = d.layers[m + 1];
            feeds_next = nx.type_layer == MYEA_LAYER_FULLY_CONNECTED && !layer_uses_norm(nx) && !L[m + 1].unit_act && !L[m + 1].noise && nx.k_sparsity == 0 &&
                         gemm_can_fuse_activation((int)nx.type_activation_function);
        }
        bool next_drop = false;
        if (feeds_next) MYEA_TRY(refresh_colscale(m + 1, &next_drop));
        MYEA_TRY(chunked(next_drop, [&](size_t t, size_t roff, size_t rows) {
            GemmParams g{};
            g.A = in + roff * In; g.lda = (long)In; g.a_k_contiguous = 1;
            g.B = parameters + l.first_connection_index; g.ldb = (long)In; g.b_k_contiguous = 1;
            g.C = o.summations + roff * H; g.ldc = (long)H;
            g.M = (int)rows; g.N = (int)H; g.K = (int)In;
            g.epilogue = EPI_FC_FORWARD;
            g.bias = layer_uses_bias(l) ? parameters + l.first_bias_connection_index : nullptr;
            if (feeds_next) {
                g.act = (int)d.layers[m + 1].type_activation_function;
                g.aux_out = L[m + 1].values + roff * H;
                g.colscale = next_drop ? L[m + 1].colscale + t * L[m + 1].AH : nullptr;
            }
            prof_begin(0);
            const int rc = launch_gemm(stream, g);
            prof_end(2.0 * (double)rows * (double)H * (double)In);
            return rc;
        }));
        values_ready = feeds_next;
    }
    DevLayer &o = L[ri];
    const float *blk = layer_outputs(last);   // a dense member's sums, a pooling member's values, an LSTM member's outputs
    if (layer_uses_norm(r)) {
        MYEA_TRY(bn_forward_all(ri, B, blk, training));
        blk = o.normalizes;
    }
    // ShakeDrop on the block's output, in place (NN/Neural_Network__Forward_Pass__Loop.cpp:4053-4078): one mask per (time step,
    // example), one draw per value (Recurrent__Forward_Pass__Dropout__ShakeDrop, NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:367-386)
    if (r.type_dropout == MYEA_DROPOUT_SHAKEDROP) {
        const size_t W = o.NH;
        float *out = const_cast<float *>(blk);
        if (state == MYEA_STATE_TRAINING) {
            if (!o.noise_uploaded) {   // masks, forward and backward draws of this pass, all time steps
                MYEA_TRY(launch_dropout_noise(stream, T * Bmax, o.noise, 0, 0.f, 1.f, dropout_seed, dropout_stream++));
                MYEA_TRY(launch_threshold(stream, T * Bmax, o.noise, r.dropout_values[0]));
                MYEA_TRY(launch_dropout_noise(stream, T * Bmax * W, o.noise + T * Bmax, 0, -1.f, 1.f, dropout_seed, dropout_stream++));
                MYEA_TRY(launch_dropout_noise(stream, T * Bmax * W, o.noise + T * Bmax + T * Bmax * W, 0, 0.f, 1.f, dropout_seed, dropout_stream++));
            }
            MYEA_TRY(chunked(false, [&](size_t, size_t roff, size_t rows) {
                return launch_shakedrop_apply(stream, rows, W, out + roff * W, o.noise + roff, o.noise + T * Bmax + roff * W, 1.f);
            }));
        } else {
            MYEA_TRY(chunked(false, [&](size_t, size_t roff, size_t rows) {
                return launch_shakedrop_apply(stream, rows, W, out + roff * W, nullptr, nullptr, 1.f - r.dropout_values[0]);
            }));
        }
    }
    const size_t na = o.In, nb = o.NH;
    const float *src = layer_outputs(o.prev);
    return chunked(false, [&](size_t, size_t roff, size_t rows) {
        float *out = o.values + roff * o.H;
        if (na >= nb) return launch_padded_add(stream, rows, o.H, src + roff * na, na, 0, blk + roff * nb, nb, -(long)o.pad, out);
        return launch_padded_add(stream, rows, o.H, blk + roff * nb, nb, 0, src + roff * na, na, -(long)o.pad, out);
    });
}

// ---- Compute__Error -------------------------------------------------------------------------------------------
// what Compute__Error, Compute__Loss and Compute__Accuracy__R share: the output layer's tensors and the staged targets
int Net::output_error_params(size_t B, const float *desired, int on_device, const char *fn, ErrorParams *out)
{
    if (!desired) { set_last_error("%s: null desired outputs", fn); return MYEA_E_INVALID; }
    if (B == 0 || B > d.batch_size) { set_last_error("%s: batch size (%zu) > maximum batch size (%u)", fn, B, d.batch_size); return MYEA_E_BATCH; }
    const size_t lo = d.n_layers - 1, T = d.number_recurrent_depth;
    const myea_layer_desc &l = d.layers[lo];
    if (l.type_layer != MYEA_LAYER_FULLY_CONNECTED) { set_last_error("%s: the output layer must be fully connected", fn); return MYEA_E_UNSUPPORTED; }
    DevLayer &o = L[lo];
    const float *dsrc = desired;
    if (!on_device) {
        MYEA_HIP_TRY(hipMemcpyAsync(stage_out, desired, B * T * o.H * sizeof(float), hipMemcpyHostToDevice, stream));
        dsrc = stage_out;
    }
    ErrorParams p{};
    p.B = B; p.T = T; p.H = o.H; p.Bmax = d.batch_size;
    p.values = o.values;
    p.pre = (layer_uses_norm(l) && l.use_layer_normalization_before_activation) ? o.normalizes : o.summations;
    p.desired = dsrc;
    p.errors = o.neuron_errors;  // AF errors are copied to the neuron errors unchanged (:136-139)
    p.act = (int)l.type_activation_function; p.steep = l.activation_steepness;
    p.unit_act = o.unit_act; p.unit_steep = o.unit_steep;
    p.loss = (int)h.type_loss_function; p.accuracy = (int)h.type_accuracy_function;
    p.accuracy_variance = h.accuracy_variance; p.bit_fail_limit = h.bit_fail_limit;
    p.first_t = T > 1 ? h.number_time_delays : 0;
    p.rnn_pre_quirk = T > 1;
    p.loss_acc = loss_acc;
    p.write_delta = 1;
    *out = p;
    return MYEA_OK;
}

int Net::compute_error(size_t B, const float *desired, int on_device)
{
    ErrorParams p;
    MYEA_TRY(output_error_params(B, desired, on_device, "Compute__Error", &p));
    // algorithmic bytes: the outputs and the desired values read once, the delta written once
    prof_begin(kProfOutputError);
    const int rc = launch_compute_error(stream, p);
    prof_end((double)B * (double)p.T * (double)p.H * sizeof(float) * 3.0);
    return rc;
}

// Compute__Loss (NN/Neural_Network__Compute__Loss__Loop.cpp:22-140): loss and accuracy of the values the last forward pass left
int Net::compute_loss(size_t B, const float *desired, int on_device)
{
    ErrorParams p;
    MYEA_TRY(output_error_params(B, desired, on_device, "Compute__Loss", &p));
    p.write_delta = 0;
    return launch_compute_error(stream, p);
}

int Net::compute_accuracy_r(size_t B, const float *desired, int on_device, float desired_mean, float predicted_mean)
{
    ErrorParams p;
    MYEA_TRY(output_error_params(B, desired, on_device, "Compute__Accuracy__R", &p));
    return launch_accuracy_r(stream, p, desired_mean, predicted_mean);
}

int Net::gather_examples(float *dst, const float *src, size_t examples, size_t row_floats, const uint64_t *index, int index_on_device, size_t B)
{
    if (!dst || !src || !index) { set_last_error("gather_examples: null argument"); return MYEA_E_INVALID; }
    const unsigned long long *dindex = reinterpret_cast<const unsigned long long *>(index);
    if (!index_on_device) {
        if (B > d.batch_size) { set_last_error("gather_examples: batch size (%zu) > maximum batch size (%u)", B, d.batch_size); return MYEA_E_BATCH; }
        for (size_t b = 0; b < B; ++b)
            if (index[b] >= examples) { set_last_error("gather_examples: index[%zu] = %llu outside the %zu examples", b, (unsigned long long)index[b], examples); return MYEA_E_INVALID; }
        MYEA_HIP_TRY(hipMemcpyAsync(index_stage, index, B * sizeof(unsigned long long), hipMemcpyHostToDevice, stream));
        dindex = index_stage;
    }
    return launch_gather_rows(stream, B, row_floats, dindex, src, dst);
}

// ---- backward ---------------------------------------------------------------------------------------------------
// What pooling layer gi hands down to its producer's `rows` rows at row offset roff, into dst; when gi is the first member of
// a residual block, plus the shortcut's share (the residual layer's errors, cropped at the padding offset).
int Net::pool_backward_with_shortcut(size_t gi, size_t rows, size_t roff, const DevLayer *shortcut, long crop, float *dst)
{
    DevLayer &on = L[gi];
    const size_t In = on.In;
    float *through = shortcut ? tmp2 + roff * In : dst;
    MYEA_TRY(launch_pool_backward(stream, pool_params(gi, rows), on.neuron_errors + roff * on.H, on.pool_index ? on.pool_index + roff * on.H : nullptr, through));
    if (shortcut) MYEA_TRY(launch_padded_add(stream, rows, In, shortcut->neuron_errors + roff * shortcut->H, shortcut->H, crop, through, In, 0, dst));
    return MYEA_OK;
}

// FF__Backward_Pass_Batch (NN/Neural_Network__Backward_Pass__OpenMP.cpp:24-155): for every layer below the
// output layer, dX = delta_next * W_next (Backward_Pass__FC, :1044-1082) and then
// Backward_Pass__Gradient__FC (:544-709): [BN after] -> act' -> [BN before].  The act' multiply is fused
// into the dX contraction's epilogue whenever it directly follows it.
int Net::backward_into_layer(size_t li, size_t B)
{
    const myea_layer_desc &l = d.layers[li];
    DevLayer &o = L[li];
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size, H = o.H;
    // next_connected_layers (Organize__Next_Layers_Connected, NN/Neural_Network.cpp:59-102): the layer after this one (after
    // this block, for a residual layer); when that is a residual layer, its shortcut AND its block's first member consume
    // this layer.  The shortcut's share (Backward_Pass__Residual, NN/Neural_Network__Backward_Pass__OpenMP.cpp:1155-1215:
    // the residual layer's errors, cropped at the padding offset) joins the contraction as its addend.
    size_t gi = l.type_layer == MYEA_LAYER_RESIDUAL ? li + l.block_depth + 1 : li + 1;
    const float *addend = nullptr, *identity = nullptr;
    const DevLayer *shortcut = nullptr;
    long ld_addend = 0, crop = 0;
    bool have_gemm = true;
    if (d.layers[gi].type_layer == MYEA_LAYER_RESIDUAL) {
        shortcut = &L[gi];
        crop = shortcut->H > H ? (long)shortcut->pad : 0;
        addend = shortcut->neuron_errors + crop;
        ld_addend = (long)shortcut->H;
        gi += 1;
        // a normalised first member hands down its normalisation errors (Backward_Pass__Residual__FC, :454-534)
        if (layer_uses_norm(d.layers[gi])) { have_gemm = false; identity = L[gi].in_errors; }
    }
    const myea_layer_desc &next = d.layers[gi];
    DevLayer &on = L[gi];
    // a pooling consumer hands its errors down through its windows instead of a contraction
    const bool pool_consumer = layer_is_pooling(next);
    if (pool_consumer) have_gemm = false;
    // what the consumer hands down: delta [T][Bmax][Out] and weights [Out][H]
    const float *delta = on.neuron_errors, *weights = parameters + next.first_connection_index;
    size_t Out = on.H;
    if (next.type_layer == MYEA_LAYER_LSTM) lstm_delta_source(gi, 0, &delta, &Out, &weights);
    const bool second_direction = next.type_layer == MYEA_LAYER_LSTM && on.lstm2 != nullptr;
    const bool is_fc = layer_is_dense(l), ind = layer_is_ind_rnn(l);
    const bool norm = is_fc && layer_uses_norm(l), before = l.use_layer_normalization_before_activation != 0;
    const bool seq_bn = T > 1 && norm && before && B == Bmax && bn_sequence_allowed() && 2 * T * H <= scratch_floats;
    const bool per_t = T > 1 && !seq_bn && (B != Bmax || norm);
    const size_t chunks = per_t ? T : 1, rows = per_t ? B : (T > 1 ? T * B : B);
    for (size_t c = 0; c < chunks; ++c) {
        const size_t roff = c * Bmax;
        GemmParams g{};
        g.A = delta + roff * Out; g.lda = (long)Out; g.a_k_contiguous = 1;
        g.B = weights; g.ldb = (long)H; g.b_k_contiguous = 0;
        g.M = (int)rows; g.N = (int)H; g.K = (int)Out;
        g.ldc = (long)H;
        g.addend = addend ? addend + roff * (size_t)ld_addend : nullptr; g.ld_addend = ld_addend;
        if (second_direction) {  // the time-reversed direction's share dG2 Win2 first; it joins the main contraction as its addend
            const float *delta2, *weights2;
            size_t out2;
            lstm_delta_source(gi, 1, &delta2, &out2, &weights2);
            GemmParams g2 = g;
            g2.A = delta2 + roff * out2; g2.lda = (long)out2; g2.B = weights2; g2.K = (int)out2;
            g2.C = tmp2 + roff * H; g2.epilogue = EPI_NONE;   // (a shortcut's share, when there is one, rides along as this launch's addend)
            prof_begin(1);
            MYEA_TRY(launch_gemm(stream, g2));
            prof_end(2.0 * (double)rows * (double)H * (double)out2);
            g.addend = tmp2 + roff * H; g.ld_addend = (long)H;
        }
        if (!is_fc) {  // an LSTM layer receives the plain delta of its cell outputs (BPTT follows), a residual layer that of its units
            g.C = o.neuron_errors + roff * H;
            g.epilogue = EPI_NONE;
            if (pool_consumer) { MYEA_TRY(pool_backward_with_shortcut(gi, rows, roff, shortcut, crop, g.C)); continue; }
            if (!have_gemm) { MYEA_TRY(launch_padded_add(stream, rows, H, shortcut->neuron_errors + roff * shortcut->H, shortcut->H, crop, identity + roff * H, H, 0, g.C)); continue; }
            prof_begin(1);
            MYEA_TRY(launch_gemm(stream, g));
            prof_end(2.0 * (double)rows * (double)H * (double)Out);
            continue;
        }
        g.act = (int)l.type_activation_function; g.steep = l.activation_steepness;
        const bool fuse = !ind && have_gemm && !o.unit_act && !o.unit_steep && gemm_can_fuse_activation(g.act);
        if (ind) {
            g.C = tmp1 + roff * H;
            g.epilogue = EPI_NONE;
        } else if (!norm) {
            g.C = (fuse ? o.neuron_errors : tmp1) + roff * H;
            g.epilogue = fuse ? EPI_FC_DERIVE : EPI_NONE; g.pre = o.summations + roff * H; g.val = o.values + roff * H;
            // this launch writes the layer's final errors: their column sums (the bias gradient's) come out with them
            if (fuse && chunks == 1 && o.bias_partials) { g.col_partials = o.bias_partials; o.bias_partial_rows = (rows + 31) / 32; o.bias_partial_batch = B; }
        } else if (before) {
            g.C = tmp1 + roff * H;
            g.epilogue = fuse ? EPI_FC_DERIVE : EPI_NONE; g.pre = o.normalizes + roff * H; g.val = o.values + roff * H;
            // the sums the normalisation's backward pass starts with leave with the contraction's tiles
            if (!seq_bn && fuse && o.norm_partials && bn_sums_from_gemm(true) && l.type_normalization == MYEA_NORMALIZATION_BATCH_NORMALIZATION && o.NH == H) {
                g.col_partials = o.norm_partials; g.hats = o.hats + roff * H;
            }
        } else {
            g.C = tmp1 + roff * H;
            g.epilogue = EPI_NONE;
        }
        if (have_gemm) {
            bool paired = false;
            GemmParams w{};
            if (pairing && chunks == 1 && !second_direction && next.type_layer == MYEA_LAYER_FULLY_CONNECTED && on.group == 0 && fc_dw_params(gi, B, &w)) {
                prof_begin(4);
                const int rc = launch_gemm_pair(stream, g, w);
                if (rc < 0) return rc;
                paired = rc == MYEA_OK;
                if (paired) {
                    prof_end(2.0 * (double)rows * (double)H * (double)Out + 2.0 * (double)w.M * (double)w.N * (double)w.K);
                    dw_done[gi] = 1;
                    if (gi < dw_zero.size()) dw_zero[gi] = 0;
                    if (early_update) MYEA_TRY(early_update_layer(gi));   // that launch was the last reader of the layer's weights in this pass
                } else prof_cancel();
            }
            if (!paired) {
                prof_begin(1);
                MYEA_TRY(launch_gemm(stream, g));
                prof_end(2.0 * (double)rows * (double)H * (double)Out);
            }
        } else if (pool_consumer) {
            MYEA_TRY(pool_backward_with_shortcut(gi, rows, roff, shortcut, crop, g.C));
        } else {
            MYEA_TRY(launch_padded_add(stream, rows, H, shortcut->neuron_errors + roff * shortcut->H, shortcut->H, crop, identity + roff * H, H, 0, g.C));
        }
        if (ind) {   // the recurrence follows for the whole sequence
            if (norm && !before) MYEA_TRY(bn_backward(li, c, rows, o.values + roff * H, tmp1 + roff * H, tmp2 + roff * H));
            continue;
        }
        if (!fuse && !(norm && !before)) {  // act' as its own kernel (Backward_Pass__FC__DF)
            MYEA_TRY(launch_activation_derive(stream, g.act, g.steep, rows * H, g.pre, g.val, tmp1 + roff * H, (norm ? tmp1 : o.neuron_errors) + roff * H,
                                              o.unit_act, o.unit_steep, H));
        }
        if (norm && before && seq_bn) {
            MYEA_TRY(bn_backward_all(li, B, o.summations, tmp1, o.neuron_errors));
        } else if (norm && before) {
            const bool sums_from_gemm = have_gemm && g.col_partials == o.norm_partials && g.col_partials != nullptr;
            MYEA_TRY(bn_backward(li, c, rows, o.summations + roff * H, tmp1 + roff * H, o.neuron_errors + roff * H, sums_from_gemm ? o.norm_partials : nullptr, (rows + 31) / 32));
        } else if (norm) {
            MYEA_TRY(bn_backward(li, c, rows, o.values + roff * H, tmp1 + roff * H, tmp2 + roff * H));
            MYEA_TRY(launch_activation_derive(stream, (int)l.type_activation_function, l.activation_steepness, rows * H,
                                              o.summations + roff * H, o.values + roff * H, tmp2 + roff * H, o.neuron_errors + roff * H, o.unit_act, o.unit_steep, H));
        }
    }
    if (ind) {
        // Backward_Pass__FC__DF_Ind_RNN for all time steps, then the normalisation in front of the activation, per time step
        IndRnnParams p{};
        p.T = T; p.B = B; p.Bmax = Bmax; p.H = H;
        p.u = parameters + l.first_connection_index + H * o.In;
        p.act = (int)l.type_activation_function; p.steep = l.activation_steepness; p.unit_act = o.unit_act; p.unit_steep = o.unit_steep;
        p.pre_afs = o.pre_afs; p.afs = o.values;
        p.dy = (norm && !before) ? tmp2 : tmp1;
        p.dafs = o.dafs_own ? o.dafs_own : o.neuron_errors;
        p.du_rows = o.du_rows;
        MYEA_TRY(launch_ind_rnn_backward(stream, p));
        o.du_rows_batch = o.du_rows ? B : 0;
        if (norm && before) MYEA_TRY(bn_backward_all(li, B, o.summations, o.dafs_own, o.neuron_errors));
    }
    return MYEA_OK;
}

// Backward_Pass__Gradient__Residual (NN/Neural_Network__Backward_Pass__OpenMP.cpp:711-950) with
// Backward_Pass__Residual__Block (:351-452) and Backward_Pass__Residual__FC (:454-534), members from the last to the first,
// each over all of its time steps before the member in front of it (Recurrent__Backward_Pass__Gradient__Residual__Layer,
// NN/Neural_Network__Recurrent_Backward_Pass__OpenMP.cpp:885-1001).
// The last member's delta is the residual layer's errors (cropped to its width), through the block-level BN backward when
// there is one.  A dense member reduces its delta to its input side: dX = delta * W, times act' of its input-side activation
// (an independently recurrent member: through its recurrence over the time steps), through its BN backward; that result IS
// the delta of the member before it (the reference copies it there), so it is written straight into that member's buffer.
// An LSTM member runs its time loop backwards and hands the member before it dG * Win.  A normalised first member keeps its
// input-side errors for the shortcut source; an un-normalised one, or an LSTM, contributes its contraction there directly
// (backward_into_layer).
int Net::backward_residual_block(size_t ri, size_t B)
{
    const myea_layer_desc &r = d.layers[ri];
    DevLayer &ro = L[ri];
    const size_t last = ri + r.block_depth, T = d.number_recurrent_depth, Bmax = d.batch_size;
    const long crop = ro.H > ro.NH ? (long)ro.pad : 0;
    // the whole sequence in one launch when the batch fills the network's rows, one launch per time step otherwise (the time
    // steps are on their own in everything that is not a recurrence)
    auto chunked = [&](auto &&launch) -> int {
        const bool split = T > 1 && B != Bmax;
        const size_t n = split ? T : 1, rows = split ? B : T * B;
        for (size_t c = n; c-- > 0;) MYEA_TRY(launch(c * Bmax, rows));
        return MYEA_OK;
    };
    // the perturbed examples' deltas times the backward draws (NN/Neural_Network__Backward_Pass__Loop.cpp:433-443)
    const bool shake = r.type_dropout == MYEA_DROPOUT_SHAKEDROP;
    {
        const bool norm = layer_uses_norm(r);
        float *to = norm ? tmp1 : L[last].neuron_errors;
        const size_t W = norm ? ro.NH : L[last].H;   // (the same width: the block's last member's)
        MYEA_TRY(chunked([&](size_t roff, size_t rows) -> int {
            MYEA_TRY(launch_padded_add(stream, rows, ro.NH, ro.neuron_errors + roff * ro.H, ro.H, crop, nullptr, 0, 0, to + roff * W));
            if (shake) MYEA_TRY(launch_shakedrop_apply(stream, rows, ro.NH, to + roff * W, ro.noise + roff, ro.noise + T * Bmax + T * Bmax * ro.NH + roff * ro.NH, 1.f));
            return MYEA_OK;
        }));
        if (norm) MYEA_TRY(bn_backward_all(ri, B, layer_outputs(last), tmp1, L[last].neuron_errors));
    }
    for (size_t m = last; m > ri; --m) {
        const myea_layer_desc &l = d.layers[m];
        DevLayer &o = L[m];
        const bool norm = layer_uses_norm(l), first = m == ri + 1;
        const size_t In = o.In, H = o.H;
        if (l.type_layer == MYEA_LAYER_LSTM) {
            MYEA_TRY(lstm_backward_layer(m, B));
            if (first) break;   // the layer in front of the block pulls dG * Win together with the shortcut's share
            // what the member before it receives: dG * Win of every time step (both directions of a two-direction member)
            MYEA_TRY(chunked([&](size_t roff, size_t rows) -> int {
                for (int direction = o.lstm2 ? 1 : 0; direction >= 0; --direction) {
                    const float *delta, *weights;
                    size_t out;
                    lstm_delta_source(m, direction, &delta, &out, &weights);
                    GemmParams g{};
                    g.A = delta + roff * out; g.lda = (long)out; g.a_k_contiguous = 1;
                    g.B = weights; g.ldb = (long)In; g.b_k_contiguous = 0;
                    g.M = (int)rows; g.N = (int)In; g.K = (int)out;
                    g.ldc = (long)In; g.epilogue = EPI_NONE;
                    g.C = (direction == 1 ? tmp2 : L[m - 1].neuron_errors) + roff * In;
                    if (direction == 0 && o.lstm2) { g.addend = tmp2 + roff * In; g.ld_addend = (long)In; }
                    prof_begin(1);
                    MYEA_TRY(launch_gemm(stream, g));
                    prof_end(2.0 * (double)rows * (double)In * (double)out);
                }
                return MYEA_OK;
            }));
            continue;
        }
        if (layer_is_pooling(l)) {   // hands its delta down through its windows (Backward_Pass__Gradient__Residual__Layer, :753-772), nothing else
            if (first) break;   // the first member: the layer in front of the block pulls it, together with the shortcut's share
            MYEA_TRY(chunked([&](size_t roff, size_t rows) -> int {
                return launch_pool_backward(stream, pool_params(m, rows), o.neuron_errors + roff * H, o.pool_index ? o.pool_index + roff * H : nullptr,
                                            L[m - 1].neuron_errors + roff * In);
            }));
            continue;
        }
        if (o.group == 1 && !norm) break;
        const bool ind = o.group == 2 && layer_is_ind_rnn(l);
        const float *prev_all = layer_outputs(o.prev);
        float *dst_all = o.group == 2 ? L[m - 1].neuron_errors : o.in_errors;
        MYEA_TRY(chunked([&](size_t roff, size_t rows) -> int {
            GemmParams g{};
            g.A = o.neuron_errors + roff * H; g.lda = (long)H; g.a_k_contiguous = 1;
            g.B = parameters + l.first_connection_index; g.ldb = (long)In; g.b_k_contiguous = 0;
            g.C = ((norm || ind) ? tmp1 : dst_all) + roff * In; g.ldc = (long)In;
            g.M = (int)rows; g.N = (int)In; g.K = (int)H;
            g.epilogue = EPI_NONE;
            bool derive_pending = false;
            if (o.group == 2 && !ind) {
                g.act = (int)l.type_activation_function; g.steep = l.activation_steepness;
                g.pre = (norm ? o.normalizes : prev_all) + roff * In;   // Layer::ptr_array_pre_activation_functions
                g.val = o.values + roff * In;
                if (!o.unit_act && !o.unit_steep && gemm_can_fuse_activation(g.act)) g.epilogue = EPI_FC_DERIVE;
                else derive_pending = true;
            }
            prof_begin(1);
            MYEA_TRY(launch_gemm(stream, g));
            prof_end(2.0 * (double)rows * (double)H * (double)In);
            if (derive_pending) MYEA_TRY(launch_activation_derive(stream, g.act, g.steep, rows * In, g.pre, g.val, g.C, g.C, o.unit_act, o.unit_steep, In));
            return MYEA_OK;
        }));
        if (ind) {
            // Backward_Pass__FC__DF_Ind_RNN over the whole sequence (:865-880): what the member hands on is the delta of its
            // pre-activations, through the input-side normalisation when there is one
            IndRnnParams p{};
            p.T = T; p.B = B; p.Bmax = Bmax; p.H = In;
            p.u = parameters + l.first_connection_index + H * In;
            p.act = (int)l.type_activation_function; p.steep = l.activation_steepness; p.unit_act = o.unit_act; p.unit_steep = o.unit_steep;
            p.pre_afs = o.pre_afs; p.afs = o.values;
            p.dy = tmp1; p.dafs = o.dafs_own;
            p.du_rows = o.du_rows;
            MYEA_TRY(launch_ind_rnn_backward(stream, p));
            o.du_rows_batch = o.du_rows ? B : 0;
            if (norm) MYEA_TRY(bn_backward_all(m, B, prev_all, o.dafs_own, dst_all));
            else MYEA_HIP_TRY(hipMemcpyAsync(dst_all, o.dafs_own, T * Bmax * In * sizeof(float), hipMemcpyDeviceToDevice, stream));
        } else if (norm) {
            MYEA_TRY(bn_backward_all(m, B, prev_all, tmp1, dst_all));
        }
    }
    return MYEA_OK;
}

int Net::bn_backward(size_t li, size_t t, size_t rows, const float *x, const float *dy, float *dx, const float *sums, size_t sum_blocks)
{
    const myea_layer_desc &l = d.layers[li];
    DevLayer &o = L[li];
    const size_t H = o.NH, roff = t * d.batch_size;
    BnBackwardParams p{};
    p.rows = rows; p.H = H; p.x = x; p.hats = o.hats + roff * H; p.dy = dy;
    p.mean = o.means + t * H; p.var = o.variances + t * H; p.scale = scale_ptr(parameters, li); p.r_corr = o.r_corrections + t * H;
    p.dscale = scale_ptr(gradient, li); p.dshift = shift_ptr(gradient, li);
    p.dx = dx;
    p.renorm = l.type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
    // algorithmic bytes: dy and x-hat read once, dx written once
    prof_begin(kProfNormalization);
    const int rc = (sums && !p.renorm) ? launch_bn_backward_from_sums(stream, p, sums, sum_blocks) : launch_bn_backward(stream, p, scratch);
    prof_end((double)rows * (double)H * sizeof(float) * 3.0);
    return rc;
}

int Net::backward_pass_and_update_derivative_weight(size_t B)
{
    dw_done.assign(d.n_layers, 0);
    // MYEA_GEMM_PAIR=0 in the environment keeps the two passes as separate launches (for A / B timing on one machine)
    static const bool pair_off = [] { const char *e = std::getenv("MYEA_GEMM_PAIR"); return e && e[0] == '0'; }();
    pairing = !pair_off;
    int rc = backward_pass(B);
    pairing = false;
    if (rc == MYEA_OK) rc = update_derivative_weight(B, 1, d.n_layers);
    if (rc == MYEA_OK && dw_beside_loop) rc = side_stream_join();
    dw_beside_loop = false;
    dw_done.assign(d.n_layers, 0);
    return rc;
}

int Net::backward_pass(size_t B)
{
    if (B == 0 || B > d.batch_size) { set_last_error("Backward_Pass: batch size (%zu) > maximum batch size (%u)", B, d.batch_size); return MYEA_E_BATCH; }
    if (state != MYEA_STATE_TRAINING) { set_last_error("Backward_Pass: can not back propagate gradient in inference mode"); return MYEA_E_STATE; }
    for (DevLayer &o : L) { o.bias_partial_rows = 0; o.du_rows_batch = 0; }   // set again by the launches that leave such sums
    bn_jobs_pending.clear();
    // the walk of FF__Backward_Pass_Batch: from a consumer gi to its producer li = previous_connected_layers[0]; once a
    // residual layer's block is done it resumes from the residual layer itself (:117-120)
    for (size_t gi = d.n_layers - 1; gi != 1; --gi) {
        const size_t li = L[gi].prev;
        MYEA_TRY(backward_into_layer(li, B));
        if (d.layers[li].type_layer == MYEA_LAYER_LSTM) {
            // The weight contractions of the consumer above need nothing the time loop of this layer produces, and the loop leaves
            // most of the matrix pipe idle: in the combined call they go to the side stream, enqueued right behind the loop so that
            // its workgroups are placed first.  MYEA_DW_BESIDE_LOOP=0 keeps them behind the loop on the one stream.
            const bool beside = pairing && dw_beside_loop_allowed(gi, li, B);
            if (beside) MYEA_HIP_TRY(hipEventRecord(fork_event, stream));
            loop_shares_device = beside;
            const int loop_rc = lstm_backward_layer(li, B);
            loop_shares_device = false;
            MYEA_TRY(loop_rc);
            if (beside) {
                MYEA_HIP_TRY(hipStreamWaitEvent(side_stream, fork_event, 0));
                std::swap(stream, side_stream);
                const int rc = update_derivative_weight_contraction(gi, B);
                std::swap(stream, side_stream);
                MYEA_HIP_TRY(hipEventRecord(join_event, side_stream));
                dw_beside_loop = true;
                MYEA_TRY(rc);
                dw_done[gi] = 1;
            }
        } else if (d.layers[li].type_layer == MYEA_LAYER_RESIDUAL) {
            MYEA_TRY(backward_residual_block(li, B));
            gi = li + 1;
        }
    }
    return flush_bn_shares();
}

// ---- Update_Derivative_Weight -----------------------------------------------------------------------------------
// FF__Update_Derivative_Weight_Batch (NN/Neural_Network__Update_Derivative_Weight__OpenMP.cpp:24-59):
// dW += delta^T X (:178-216) with X = the previous layer's post-dropout outputs, db += column sums (:218-242).
// slabs of the split-K form of a fully-connected layer's weight gradient; 1 = the plain accumulating contraction
static int fc_dw_slabs(size_t H, size_t In, size_t rows, size_t first_connection_index)
{
    (void)first_connection_index;
    if (rows > 0x7fffffffu) return 1;
    const int narrow = narrow_dw_slabs(H, In, rows);   // a narrow layer's kernel of its own: always through slabs
    if (narrow > 0) return narrow > 1 ? narrow : 2;    // (room for two, so that "more than one slab" still says "through slabs")
    return gemm_split_k((int)H, (int)In, (int)rows);
}

// the weight gradient of fully-connected layer li as one accumulating contraction dW += delta^T X (false when it takes the
// per-time-step or the split-K form instead)
bool Net::fc_dw_params(size_t li, size_t B, GemmParams *out)
{
    const myea_layer_desc &l = d.layers[li];
    DevLayer &o = L[li];
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size, In = o.In, H = o.H;
    if (T > 1 && B != Bmax) return false;
    const size_t rows = T > 1 ? T * B : B;
    if (dw_slabs && fc_dw_slabs(H, In, rows, l.first_connection_index) > 1) return false;
    const float *x = layer_outputs(o.prev);
    if (o.group == 2) x = o.values;
    else if (o.group == 1 && layer_uses_norm(l)) x = o.normalizes;
    GemmParams g{};
    g.A = o.neuron_errors; g.lda = (long)H; g.a_k_contiguous = 0;
    g.B = x; g.ldb = (long)In; g.b_k_contiguous = 0;
    g.C = gradient + l.first_connection_index; g.ldc = (long)In;
    g.M = (int)H; g.N = (int)In; g.K = (int)rows;
    g.accumulate = 1; g.c_is_zero = dw_may_store(li) ? 1 : 0; g.epilogue = EPI_NONE;
    *out = g;
    return true;
}

bool Net::dw_may_store(size_t li) const
{
    static const bool off = [] { const char *e = std::getenv("MYEA_DW_STORE"); return e && e[0] == '0'; }();
    return !off && li < dw_zero.size() && dw_zero[li];
}

// the weight contraction(s) of layer li: dW += delta^T X (:178-216); LSTM layers: their input and recurrent weights
int Net::update_derivative_weight_contraction(size_t li, size_t B)
{
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size;
    const bool per_t = T > 1 && B != Bmax;
    const size_t chunks = per_t ? T : 1, rows = per_t ? B : (T > 1 ? T * B : B);
    const myea_layer_desc &l = d.layers[li];
    if (li < dw_done.size() && dw_done[li]) return MYEA_OK;   // rode along with the delta's contraction, or ran beside a time loop, in this pass
    if (l.type_layer == MYEA_LAYER_LSTM) return lstm_update_derivative_weight(li, B, false);
    if (l.type_layer == MYEA_LAYER_RESIDUAL || layer_is_pooling(l)) return MYEA_OK;  // own no connection (:31-36)
    DevLayer &o = L[li];
    const size_t In = o.In, H = o.H;
    // Layer::ptr_array_pre_summations: the operand the weights were applied to (NN/Neural_Network__Ordered.cpp:96-141)
    const float *x = layer_outputs(o.prev);
    if (o.group == 2) x = o.values;
    else if (o.group == 1 && layer_uses_norm(l)) x = o.normalizes;
    for (size_t c = 0; c < chunks; ++c) {
        const size_t roff = c * Bmax;
        GemmParams g{};
        g.A = o.neuron_errors + roff * H; g.lda = (long)H; g.a_k_contiguous = 0;
        g.B = x + roff * In; g.ldb = (long)In; g.b_k_contiguous = 0;
        g.C = gradient + l.first_connection_index; g.ldc = (long)In;
        g.M = (int)H; g.N = (int)In; g.K = (int)rows;
        g.accumulate = 1; g.c_is_zero = dw_may_store(li) ? 1 : 0; g.epilogue = EPI_NONE;
        int slabs = dw_slabs ? fc_dw_slabs(H, In, rows, l.first_connection_index) : 1;
        const int narrow = dw_slabs ? narrow_dw_slabs(H, In, rows) : 0;
        if (slabs > 1) { g.C = dw_slabs; g.accumulate = 0; g.c_is_zero = 0; g.split_k = slabs; g.split_k_slab = (long)(H * In); }
        if (li < dw_zero.size()) dw_zero[li] = 0;   // from here on the slice holds this product, stored or added from the slabs
        prof_begin(2);
        // a narrow layer over all of its rows: the slabs wait in the layer's slice for the one launch that adds every layer's
        const bool later = defer_folds && narrow > 0 && chunks == 1 && narrow_slabs && narrow_slab_at[li] != SIZE_MAX;
        float *const slabs_at = later ? narrow_slabs + narrow_slab_at[li] : dw_slabs;
        if (narrow > 0) { slabs = narrow; MYEA_TRY(launch_narrow_dw(stream, g.A, g.B, slabs_at, H, In, rows)); }
        else MYEA_TRY(launch_gemm(stream, g));
        if (later) fold_pending.push_back(SlabFoldJob{slabs_at, gradient + l.first_connection_index, (unsigned)(H * In), (unsigned)slabs});
        else if (slabs > 1 || narrow > 0) MYEA_TRY(launch_slab_sum_add(stream, H * In, slabs, dw_slabs, gradient + l.first_connection_index, narrow > 0));
        prof_end(2.0 * (double)rows * (double)H * (double)In);
    }

    return MYEA_OK;
}

// May the weight contractions of layer gi run on the side stream beside the backward time loop of LSTM layer li?  Where nothing
// is shared and it was measured to pay: a one-direction loop (a two-direction layer uses the side stream itself) under an
// LSTM consumer, whose two long contractions write packed slabs of their own.  (A dense consumer's single contraction hides
// less than the loop loses by sharing the device: 3.93 against 3.90 ms per step on 2 x LSTM-512.)
bool Net::dw_beside_loop_allowed(size_t gi, size_t li, size_t B)
{
    static const bool off = [] { const char *e = std::getenv("MYEA_DW_BESIDE_LOOP"); return e && e[0] == '0'; }();
    if (off || !side_stream || d.number_recurrent_depth < 2 || B != d.batch_size) return false;
    if (L[li].lstm2 || L[gi].lstm2 || (gi < dw_done.size() && dw_done[gi])) return false;
    if (d.layers[gi].type_layer != MYEA_LAYER_LSTM || !L[li].lstm) return false;
    // ... and a loop that leaves at least half of the compute units without a workgroup.  One that fills the device is faster
    // alone in its column form than in the k form beside the contractions, by more than those then hide (2 x LSTM-512 at a
    // batch of 256: 3.66 against 3.70 ms per step).
    return lstm_backward_loop_leaves_room(li, B);
}

int Net::update_derivative_weight(size_t B, size_t first, size_t end)
{
    if (first < 1 || end > d.n_layers || first > end) { set_last_error("Update_Derivative_Weight: layer range [%zu, %zu) invalid", first, end); return MYEA_E_INVALID; }
    if (B == 0 || B > d.batch_size) { set_last_error("Update_Derivative_Weight: batch size (%zu) > maximum batch size (%u)", B, d.batch_size); return MYEA_E_BATCH; }
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size;
    const bool per_t = T > 1 && B != Bmax;
    const size_t chunks = per_t ? T : 1, rows = per_t ? B : (T > 1 ? T * B : B);
    fold_pending.clear();
    // The column reductions (biases, LSTM peepholes, self weights of independently recurrent layers) read deltas that
    // are complete before this call and write gradient slots no contraction touches; slots shared between layers (the
    // LSTM bias addressing reaches into the next layers' biases) are added to in the layers' order, on one stream.
    auto reductions = [&]() -> int {
        for (size_t li = first; li < end; ++li) {
            const myea_layer_desc &l = d.layers[li];
            if (l.type_layer == MYEA_LAYER_LSTM) { MYEA_TRY(lstm_update_derivative_weight(li, B, true)); continue; }
            if (!layer_is_dense(l)) continue;
            DevLayer &o = L[li];
            if (layer_uses_bias(l))
                for (size_t c = 0; c < chunks; ++c) {
                    prof_begin(kProfBiasGradient);
                    if (chunks == 1 && o.bias_partial_rows == (rows + 31) / 32 && o.bias_partial_batch == B) {
                        MYEA_TRY(launch_column_sum_final(stream, o.H, o.bias_partial_rows, o.bias_partials, gradient + l.first_bias_connection_index, 1));
                        prof_end((double)o.bias_partial_rows * (double)o.H * sizeof(float));
                    } else {
                        MYEA_TRY(launch_column_sum(stream, rows, o.H, o.neuron_errors + c * Bmax * o.H, gradient + l.first_bias_connection_index, 1, scratch));
                        prof_end((double)rows * (double)o.H * sizeof(float));
                    }
                }
            // the self weights: as many as the layer has recurrent units - its width, a block member's fan-in, none for a block's first member
            if (layer_is_ind_rnn(l) && o.group != 1) {
                const size_t units = o.group ? o.AH : o.H;
                float *du = gradient + l.first_connection_index + o.H * o.In;
                // the backward time loop left every example's share: they are added with the narrow layers' slabs, one launch for all
                if (defer_folds && fold_jobs && o.du_rows && o.du_rows_batch == B && T > 1) fold_pending.push_back(SlabFoldJob{o.du_rows, du, (unsigned)units, (unsigned)B});
                else MYEA_TRY(launch_ind_rnn_self_weight_gradient(stream, T, B, Bmax, units, o.values, o.dafs_own ? o.dafs_own : o.neuron_errors, du, scratch));
            }
        }
        return MYEA_OK;
    };
    // alternate: narrow layers, whose slabs wait in slices of their own, take turns on the two streams - each is a launch of a few
    // dozen workgroups and a chain of them on one stream leaves most of the device idle
    auto contractions = [&](bool alternate) -> int {
        bool on_side = false;
        for (size_t li = first; li < end; ++li) {
            const bool done_before = li < dw_done.size() && dw_done[li];
            const bool own_slice = alternate && !done_before && chunks == 1 && defer_folds && narrow_slabs && li < narrow_slab_at.size() &&
                                   narrow_slab_at[li] != SIZE_MAX && layer_is_dense(d.layers[li]) && narrow_dw_slabs(L[li].H, L[li].In, rows) > 0;
            if (own_slice && on_side) {
                std::swap(stream, side_stream);
                const int rc = update_derivative_weight_contraction(li, B);
                std::swap(stream, side_stream);
                MYEA_TRY(rc);
            } else {
                MYEA_TRY(update_derivative_weight_contraction(li, B));
            }
            if (own_slice) on_side = !on_side;
            // the combined call: every delta has been handed down by now, so the layer's weights may take their step beside the
            // contractions of the layers that follow
            if (early_update && !done_before) MYEA_TRY(early_update_layer(li));
        }
        return MYEA_OK;
    };
    bool any_lstm = false;
    for (size_t li = 1; li < d.n_layers; ++li) any_lstm = any_lstm || d.layers[li].type_layer == MYEA_LAYER_LSTM;
    if (any_lstm || !side_stream) {
        // beside the split-K contractions of LSTM layers the long reductions over T x batch rows were measured to cost
        // more than they hide: one stream, contractions first
        MYEA_TRY(contractions(false));
        MYEA_TRY(reductions());
        return flush_slab_folds();
    }
    // memory-bound reductions on the side stream beside the matrix-pipe-bound contractions, and every other narrow contraction
    MYEA_HIP_TRY(hipEventRecord(fork_event, stream));
    MYEA_HIP_TRY(hipStreamWaitEvent(side_stream, fork_event, 0));
    std::swap(stream, side_stream);
    int rc = reductions();
    std::swap(stream, side_stream);
    if (rc == MYEA_OK) rc = contractions(true);
    const hipError_t e = hipEventRecord(join_event, side_stream);   // the main stream goes on behind the side stream, whatever else happened
    const int joined = e == hipSuccess ? side_stream_join() : MYEA_E_DEVICE;
    if (e != hipSuccess && rc == MYEA_OK) set_last_error("hipEventRecord: %s", hipGetErrorString(e));
    MYEA_TRY(rc);
    MYEA_TRY(joined);
    return flush_slab_folds();
}

// Update_Derivative_Weight without any buffer of the library's own behind its kernels: the column reductions' partial
// sums, the split-K slabs of narrow fully-connected layers and the packed weight-gradient slabs of the LSTM layers are
// carved out of the static device array (in this order, each piece a multiple of 64 floats).  Same results as
// update_derivative_weight (the same additions in the same order; a narrow layer's slabs are added by a launch of the layer's own
// instead of one launch for all layers).  Nothing is allocated or freed, and the call never waits for the stream.  Every piece is written before it is read within
// the call, so what an earlier call left in the array does not matter; calls that overlap on one device (two networks
// on two streams) would share the array and race.
int Net::update_derivative_weight_no_alloc(size_t B, size_t first, size_t end)
{
    auto round_up = [](size_t n) { return (n + 63) / 64 * 64; };
    const size_t need = round_up(scratch_floats) + round_up(dw_slab_floats) + lstm_gradient_slab_floats();
    if (need > kStaticScratchFloats) {
        set_last_error("Update_Derivative_Weight (no allocation): this network's kernels need %zu bytes of scratch memory, the static buffer holds %zu",
                       need * sizeof(float), kStaticScratchFloats * sizeof(float));
        return MYEA_E_INVALID;
    }
    if (!static_scratch) { set_last_error("Update_Derivative_Weight (no allocation): the static buffer's address was not resolved"); return MYEA_E_DEVICE; }
    float *const own_scratch = scratch, *const own_slabs = dw_slabs;
    float *at = static_scratch;
    scratch = at; at += round_up(scratch_floats);
    if (own_slabs) dw_slabs = at;
    at += round_up(dw_slab_floats);
    defer_folds = false;   // a narrow layer's slabs are added right behind its contraction: no table to upload, no wait for the stream
    lstm_bind_gradient_slabs(at);
    const bool was_profiling = profiling;
    profiling = false;   // the profiling taps create events on demand
    const int rc = update_derivative_weight(B, first, end);
    profiling = was_profiling;
    scratch = own_scratch; dw_slabs = own_slabs; defer_folds = true;
    lstm_bind_gradient_slabs(nullptr);
    return rc;
}

// Per-unit activation arrays (struct AF_unit: ptr_type_activation_function / ptr_activation_steepness).  With them the
// activation can no longer ride in a contraction's epilogue; it runs as its own kernel reading the arrays per column.
int Net::set_unit_activations(size_t li, const uint32_t *types, const float *steep, size_t count)
{
    if (li == 0 || li >= d.n_layers || !layer_is_dense(d.layers[li])) { set_last_error("set_unit_activations: layer %zu is not a fully-connected hidden / output layer", li); return MYEA_E_INVALID; }
    DevLayer &o = L[li];
    if (d.layers[li].type_activation_function == MYEA_AF_SOFTMAX) { set_last_error("set_unit_activations: layer %zu is a softmax layer", li); return MYEA_E_INVALID; }
    if ((types || steep) && count != o.AH) { set_last_error("set_unit_activations: layer %zu has %zu activation units, got %zu", li, o.AH, count); return MYEA_E_INVALID; }
    if (types)
        for (size_t j = 0; j < count; ++j)
            if (types[j] == MYEA_AF_NONE || types[j] >= MYEA_AF_LENGTH || types[j] == MYEA_AF_SOFTMAX) { set_last_error("set_unit_activations: unit %zu: activation %u invalid", j, types[j]); return MYEA_E_INVALID; }
    MYEA_HIP_TRY(hipStreamSynchronize(stream));
    if (o.unit_act) { (void)hipFree(o.unit_act); o.unit_act = nullptr; }
    if (o.unit_steep) { (void)hipFree(o.unit_steep); o.unit_steep = nullptr; }
    if (types) {
        void *q = nullptr;
        MYEA_HIP_TRY(hipMalloc(&q, count * sizeof(int)));
        o.unit_act = static_cast<int *>(q);
        MYEA_HIP_TRY(hipMemcpy(o.unit_act, types, count * sizeof(int), hipMemcpyHostToDevice));
    }
    if (steep) {
        MYEA_TRY(dev_alloc(&o.unit_steep, count));
        MYEA_HIP_TRY(hipMemcpy(o.unit_steep, steep, count * sizeof(float), hipMemcpyHostToDevice));
    }
    return MYEA_OK;
}

// ---- Update_Parameter ------------------------------------------------------------------------------------------------
// Update_Parameter__OpenMP (NN/Neural_Network.cpp:4727-4828): [merge: one accumulator here] -> clip by global norm
// over all P (NN/Neural_Network__Clip_Gradient.cpp:81-94) -> optimizer.  The clip scale is applied inside the
// optimizer's gradient read instead of a separate pass over the gradient.
// Clear_Optimizer (NN/Train.cpp:128-263): the state of the CURRENT optimizer only - gradient descent its previous deltas when
// it has a momentum; iRPROP+ its two losses (to the largest float), previous derivatives, steps (to rprop_delta_zero) and
// deltas; Adam and AdaBound the two moments, AMSGrad and AMSBound the maximum too, NosAdam the moments and its running sum -
// then optimizer_time_step = 0, epoch_time_step = 1 whatever the optimizer.
int Net::clear_optimizer()
{
    const size_t P = d.total_parameters;
    auto zero = [&](int kind) -> int { MYEA_HIP_TRY(hipMemsetAsync(opt[kind], 0, P * sizeof(float), stream)); return MYEA_OK; };
    switch (h.type_optimizer_function) {
    case MYEA_OPTIMIZER_NONE: break;
    case MYEA_OPTIMIZER_GD:
        if (h.learning_momentum != 0.f) MYEA_TRY(zero(MYEA_STATE_PREVIOUS_DELTA));
        break;
    case MYEA_OPTIMIZER_IRPROP_PLUS:
        h.loss_rprop = FLT_MAX;
        h.previous_loss_rprop = FLT_MAX;
        MYEA_TRY(zero(MYEA_STATE_PREVIOUS_DERIVATIVES));
        MYEA_TRY(launch_fill(stream, opt[MYEA_STATE_PREVIOUS_STEPS], P, h.rprop_delta_zero));
        MYEA_TRY(zero(MYEA_STATE_PREVIOUS_DELTA));
        break;
    case MYEA_OPTIMIZER_AMSBOUND:
    case MYEA_OPTIMIZER_AMSGRAD:
        MYEA_TRY(zero(MYEA_STATE_FIRST_MOMENT)); MYEA_TRY(zero(MYEA_STATE_SECOND_MOMENT)); MYEA_TRY(zero(MYEA_STATE_SECOND_MOMENT_HAT));
        break;
    case MYEA_OPTIMIZER_ADABOUND:
    case MYEA_OPTIMIZER_ADAM:
        MYEA_TRY(zero(MYEA_STATE_FIRST_MOMENT)); MYEA_TRY(zero(MYEA_STATE_SECOND_MOMENT));
        break;
    case MYEA_OPTIMIZER_NOSADAM:
        MYEA_TRY(zero(MYEA_STATE_FIRST_MOMENT)); MYEA_TRY(zero(MYEA_STATE_SECOND_MOMENT));
        h.adam_previous_beta2 = 0.f;
        break;
    default:
        std::fprintf(stderr, "Clear_Optimizer: ERROR: Can not reset the optimizer parameters with (%u) as the current optimizer.\n", h.type_optimizer_function);
        break;
    }
    h.optimizer_time_step = 0.f;
    h.epoch_time_step = 1.f;
    return MYEA_OK;
}

// Warm_Restarts_Decay (NN/Train.cpp:266-283): cosine-annealed rate from the step count before this update; at the end of
// a cycle the optimizer is cleared, the cycle lengthens and its maximum rate decays.
float Net::warm_restarts_decay(int *rc)
{
    const float lr = h.warm_restarts_minimum_learning_rate
                     + 0.5f * (h.warm_restarts_maximum_learning_rate - h.warm_restarts_minimum_learning_rate)
                           * (1.f + std::cos(h.optimizer_time_step / h.warm_restarts_T_i * 3.14159265358979323846f));
    *rc = MYEA_OK;
    if (h.optimizer_time_step >= h.warm_restarts_T_i) {
        *rc = clear_optimizer();
        h.warm_restarts_T_i *= h.warm_restarts_multiplier;
        h.warm_restarts_maximum_learning_rate = std::max(h.warm_restarts_maximum_learning_rate * h.warm_restarts_decay_learning_rate,
                                                         h.warm_restarts_minimum_learning_rate);
    }
    return lr;
}

// The vectors Update_Weight_Regularization__Max_Norm_Constraints walks with (0, total_weights)
// (NN/Neural_Network__Regularization__Max_Norm_Constraints.cpp:147-332): one per fully-connected neuron (hidden and output
// layers); per LSTM block the cell-input feed-forward / recurrent vectors of each cell, then the three gates' feed-forward,
// recurrent and peephole vectors.  The LSTM tests are `first index > start`: a vector at flat index 0 is skipped.
int Net::build_max_norm_segments()
{
    if (seg_first) return MYEA_OK;
    std::vector<unsigned long long> first;
    std::vector<unsigned> len;
    for (size_t li = 1; li < d.n_layers; ++li) {
        const myea_layer_desc &l = d.layers[li];
        const size_t In = L[li].In;
        if (layer_is_dense(l)) {   // neuron units; an independently recurrent layer's self weights are not among them
            for (size_t o = 0; o < L[li].H; ++o) { first.push_back(l.first_connection_index + o * In); len.push_back((unsigned)In); }
        } else if (l.type_layer == MYEA_LAYER_LSTM) {
            const size_t K = l.n_units, cpb = l.n_cells_per_block, C = K * cpb;
            const size_t per_block = cpb * (In + C) + 3 * In + 3 * C + 3 * cpb;
            const size_t blocks = l.use_bidirectional ? 2 * K : K;
            for (size_t k = 0; k < blocks; ++k) {
                size_t at = l.first_connection_index + k * per_block;
                auto push = [&](size_t n) { if (at != 0 && n != 0) { first.push_back(at); len.push_back((unsigned)n); } at += n; };
                for (size_t j = 0; j < cpb; ++j) { push(In); push(C); }
                for (int g = 0; g < 3; ++g) push(In);
                for (int g = 0; g < 3; ++g) push(C);
                for (int g = 0; g < 3; ++g) push(cpb);
            }
        }
    }
    n_segments = first.size();
    longest_segment = 0;
    for (unsigned v : len) longest_segment = std::max(longest_segment, v);
    void *q = nullptr;
    MYEA_HIP_TRY(hipMalloc(&q, std::max<size_t>(1, n_segments) * sizeof(unsigned long long)));
    seg_first = static_cast<unsigned long long *>(q);
    MYEA_HIP_TRY(hipMalloc(&q, std::max<size_t>(1, n_segments) * sizeof(unsigned)));
    seg_len = static_cast<unsigned *>(q);
    if (n_segments) {
        MYEA_HIP_TRY(hipMemcpy(seg_first, first.data(), n_segments * sizeof(unsigned long long), hipMemcpyHostToDevice));
        MYEA_HIP_TRY(hipMemcpy(seg_len, len.data(), n_segments * sizeof(unsigned), hipMemcpyHostToDevice));
    }
    return MYEA_OK;
}

// Update_Parameter (NN/Neural_Network.cpp:4722-4911).  The L1 / L2 gradient terms are called there with (batch size, 0,
// total weights) where the callee expects (start, end, batch size) - both loops are empty
// (NN/Neural_Network__Regularization__L1.cpp:98-128), so they add nothing here either.
int Net::update_prepare(size_t B, size_t training_size, UpdateParams *out, double *out_bytes_per_param)
{
    const uint32_t kind = h.type_optimizer_function;
    switch (kind) {
    case MYEA_OPTIMIZER_GD: case MYEA_OPTIMIZER_ADAM: case MYEA_OPTIMIZER_AMSGRAD: case MYEA_OPTIMIZER_ADABOUND:
    case MYEA_OPTIMIZER_AMSBOUND: case MYEA_OPTIMIZER_NOSADAM: case MYEA_OPTIMIZER_IRPROP_PLUS: break;
    default:
        set_last_error("Update_Parameter: optimizer %u is not on this path", kind);
        return MYEA_E_UNSUPPORTED;
    }
    if (training_size == 0 && h.use_normalized_weight_decay && h.regularization__weight_decay != 0.f) {
        set_last_error("Update_Parameter: normalized weight decay needs the training-set size");
        return MYEA_E_INVALID;
    }
    // the scalars as they are before this update, until it is known to have run (resident_check)
    if (update_history.size() >= 1024) update_history.erase(update_history.begin(), update_history.begin() + 512);
    update_history.push_back(UpdateSnapshot{updates_enqueued++, h});
    UpdateParams p{};
    p.optimizer = (int)kind;
    p.n = d.total_parameters; p.n_weights = d.total_weights;
    p.w = parameters; p.g = gradient;
    p.grad_scale = 1.f;
    p.fault = fault;
    if (h.use_clip_gradient) { p.norm_sq = scratch; p.clip = h.clip_gradient; }   // the caller leaves the gradient's sum of squares there
    const bool rprop = kind == MYEA_OPTIMIZER_IRPROP_PLUS, gd = kind == MYEA_OPTIMIZER_GD;
    float scale = 1.f;
    if (h.use_Warm_Restarts && !rprop) {
        int rc = MYEA_OK;
        scale = warm_restarts_decay(&rc) / (gd ? h.learning_rate : h.adam_learning_rate);
        if (rc != MYEA_OK) return rc;
    }
    if (!rprop) h.optimizer_time_step += 1.f;
    const float ts = h.optimizer_time_step;
    // Normalized_Weight_Decay (NN/Train.cpp:285-286); only the gradient-descent family scales it by the warm-restart factor
    p.wd = h.use_normalized_weight_decay
               ? h.regularization__weight_decay * std::sqrt((float)B / ((float)training_size * h.epoch_time_step))
               : h.regularization__weight_decay;
    if (h.regularization__weight_decay == 0.f) p.wd = 0.f;
    double bytes_per_param = 16;
    if (gd) {
        p.lr = scale * h.learning_rate; p.mu = h.learning_momentum;
        p.wd *= scale;
        p.variant = h.learning_momentum != 0.f ? (h.use_Nesterov ? 2 : 1) : 0;
        p.s0 = opt[MYEA_STATE_PREVIOUS_DELTA];
        bytes_per_param = p.variant ? 24 : 16;
    } else if (rprop) {
        p.lr = h.rprop_increase_factor; p.mu = h.rprop_decrease_factor;
        p.lower = h.rprop_delta_min; p.upper = h.rprop_delta_max;
        p.beta1 = h.loss_rprop > h.previous_loss_rprop ? 1.f : 0.f;
        p.wd = 0.f;
        p.s0 = opt[MYEA_STATE_PREVIOUS_DELTA]; p.s1 = opt[MYEA_STATE_PREVIOUS_STEPS]; p.s2 = opt[MYEA_STATE_PREVIOUS_DERIVATIVES];
        bytes_per_param = 40;
    } else {
        const float lr = scale * h.adam_learning_rate;
        p.beta1 = h.adam_beta1; p.beta2 = h.adam_beta2; p.eps = h.adam_epsilon;
        // in float throughout, as NN/Neural_Network__Adam.cpp:58 evaluates it with T_ = float
        p.lr_t = h.use_adam_bias_correction ? lr * std::sqrt(1.f - std::pow(h.adam_beta2, ts)) / (1.f - std::pow(h.adam_beta1, ts)) : lr;
        p.lower = scale * h.learning_rate_final * (1.f - 1.f / (h.learning_gamma * ts + 1.f));
        p.upper = scale * h.learning_rate_final * (1.f + 1.f / (h.learning_gamma * ts));
        if (kind == MYEA_OPTIMIZER_NOSADAM) {
            // the second moment decays with beta2_t = S / (S + t^-gamma), S the sum of the earlier t^-gamma; the bias
            // correction above keeps the plain beta2 (NN/Neural_Network__NosAdam.cpp:57-70)
            const float pg = std::pow(ts, -h.adam_gamma);
            p.beta2 = h.adam_previous_beta2 / (h.adam_previous_beta2 + pg);
            h.adam_previous_beta2 += pg;
        }
        p.s0 = opt[MYEA_STATE_FIRST_MOMENT]; p.s1 = opt[MYEA_STATE_SECOND_MOMENT]; p.s2 = opt[MYEA_STATE_SECOND_MOMENT_HAT];
        bytes_per_param = (kind == MYEA_OPTIMIZER_AMSGRAD || kind == MYEA_OPTIMIZER_AMSBOUND) ? 40 : 32;
    }
    *out = p;
    *out_bytes_per_param = bytes_per_param;
    return MYEA_OK;
}

// the elementwise update of [first, first + count) of the flat vectors; first a multiple of 4 (the kernels move 16 bytes per lane)
int Net::update_range(const UpdateParams &whole, size_t first, size_t count, double bytes_per_param, bool last)
{
    if (count == 0 && !last) return MYEA_OK;
    UpdateParams p = whole;
    p.applied = last ? updates_applied : nullptr;   // the range that completes the update counts it
    p.n = count;
    p.n_weights = whole.n_weights > first ? std::min(count, whole.n_weights - first) : 0;
    p.w += first; p.g += first;
    if (p.s0) p.s0 += first;
    if (p.s1) p.s1 += first;
    if (p.s2) p.s2 += first;
    prof_begin(3);
    const int rc = launch_update(stream, p);
    prof_end(bytes_per_param * (double)count);
    return rc;
}

int Net::update_finish()
{
    gradient_known_zero(true);   // the update zeroed every element it read
    if (h.regularization__max_norm_constraints != 0.f) {
        MYEA_TRY(build_max_norm_segments());
        MYEA_TRY(launch_max_norm(stream, n_segments, seg_first, seg_len, longest_segment, h.regularization__max_norm_constraints, parameters));
    }
    // Update_Weight_Regularization__Constraint_Recurrent_Weight (NN/Neural_Network__Regularization__Constraint_Recurrent_Weight.cpp:
    // 289-333): the self weights of the independently recurrent hidden layers clipped to their bounds
    if (!clip_ranges_built) {   // the layers' bounds are part of the description: one table for the network's life
        std::vector<ClipRange> ranges;
        for (size_t li = 1; li + 1 < d.n_layers; ++li) {
            const myea_layer_desc &l = d.layers[li];
            if (!layer_is_ind_rnn(l) || L[li].group == 1 || (l.constraint_recurrent_weight_lower_bound == 0.f && l.constraint_recurrent_weight_upper_bound == 0.f)) continue;
            const size_t units = L[li].group ? L[li].AH : L[li].H;
            ranges.push_back(ClipRange{(unsigned long long)(l.first_connection_index + L[li].H * L[li].In), (unsigned)units,
                                       l.constraint_recurrent_weight_lower_bound, l.constraint_recurrent_weight_upper_bound});
            longest_clip_range = std::max(longest_clip_range, units);
        }
        n_clip_ranges = ranges.size();
        if (n_clip_ranges) {
            void *q = nullptr;
            MYEA_HIP_TRY(hipMalloc(&q, n_clip_ranges * sizeof(ClipRange)));
            clip_ranges = static_cast<ClipRange *>(q);
            MYEA_HIP_TRY(hipMemcpy(clip_ranges, ranges.data(), n_clip_ranges * sizeof(ClipRange), hipMemcpyHostToDevice));
        }
        clip_ranges_built = true;
    }
    MYEA_TRY(launch_clip_ranges(stream, clip_ranges, n_clip_ranges, longest_clip_range, parameters));
    return lstm_parameters_changed();  // refresh the packed gate matrices
}

int Net::update_parameter(size_t B, size_t training_size)
{
    UpdateParams p{};
    double bytes_per_param = 0;
    MYEA_TRY(update_prepare(B, training_size, &p, &bytes_per_param));
    if (h.use_clip_gradient) MYEA_TRY(launch_sum_squares(stream, p.n, gradient, scratch + 16, scratch));
    MYEA_TRY(update_range(p, 0, p.n, bytes_per_param, true));
    return update_finish();
}

// MYEA_EARLY_UPDATE=0 in the environment keeps the update behind the whole backward pass.  Updating a layer early needs an
// update that is elementwise with scalars known up front: no clipping by the gradient's global norm, no iRPROP (whose
// step follows the loss).
bool Net::early_update_allowed() const
{
    static const bool off = [] { const char *e = std::getenv("MYEA_EARLY_UPDATE"); return e && e[0] == '0'; }();
    // ... and no resident time loop in the pass: one that gives up after a layer above it has taken its step would leave the
    // network half updated; without LSTM layers only a forward contraction can give up, before any update of its step
    return !off && side_stream && !resident_sync && !h.use_clip_gradient && h.type_optimizer_function != MYEA_OPTIMIZER_IRPROP_PLUS;
}

// The weights of fully-connected layer li: gradient complete, no reader left in this pass.  Their update goes to the side
// stream behind what the main stream has enqueued so far.
int Net::early_update_layer(size_t li)
{
    const myea_layer_desc &l = d.layers[li];
    if (l.type_layer != MYEA_LAYER_FULLY_CONNECTED) return MYEA_OK;
    const size_t first = l.first_connection_index, count = L[li].H * L[li].In;
    // A short range's update hides less than its launch, its two events and what it takes from the kernels it runs beside
    // cost: 8 x FC-2048 (4.2 M weights a layer, Nesterov) 1.481 ms a step against 1.473 with one update at the end; 4 x FC-4096
    // (16.8 M, Adam) 3.64 against 3.74.  MYEA_EARLY_UPDATE_MIN sets another least size, in weights.
    const char *e = std::getenv("MYEA_EARLY_UPDATE_MIN");   // read at every call: a test lowers it for one network
    const size_t least = e ? (size_t)std::strtoull(e, nullptr, 10) : (size_t)1 << 23;
    if ((first & 3) || (count & 3) || count < least || count == 0) return MYEA_OK;
    MYEA_HIP_TRY(hipEventRecord(update_event, stream));
    MYEA_HIP_TRY(hipStreamWaitEvent(side_stream, update_event, 0));
    std::swap(stream, side_stream);
    const int rc = update_range(*early_update, first, count, early_bytes_per_param, false);
    std::swap(stream, side_stream);
    MYEA_TRY(rc);
    early_ranges.emplace_back(first, first + count);
    return MYEA_OK;
}

int Net::backward_pass_update_derivative_weight_and_update_parameter(size_t B, size_t training_size)
{
    if (!early_update_allowed()) {
        MYEA_TRY(backward_pass_and_update_derivative_weight(B));
        return update_parameter(B, training_size);
    }
    if (B == 0 || B > d.batch_size) { set_last_error("Backward_Pass: batch size (%zu) > maximum batch size (%u)", B, d.batch_size); return MYEA_E_BATCH; }
    if (state != MYEA_STATE_TRAINING) { set_last_error("Backward_Pass: can not back propagate gradient in inference mode"); return MYEA_E_STATE; }
    UpdateParams p{};
    MYEA_TRY(update_prepare(B, training_size, &p, &early_bytes_per_param));
    early_ranges.clear();
    early_update = &p;
    int rc = backward_pass_and_update_derivative_weight(B);
    early_update = nullptr;
    if (!early_ranges.empty()) {   // the main stream goes on behind the early updates, whatever else happened
        const hipError_t e = hipEventRecord(join_event, side_stream);
        const int joined = e == hipSuccess ? side_stream_join() : MYEA_E_DEVICE;
        if (e != hipSuccess && rc == MYEA_OK) set_last_error("hipEventRecord: %s", hipGetErrorString(e));
        if (rc == MYEA_OK) rc = joined;
    }
    if (rc != MYEA_OK) { early_ranges.clear(); return rc; }
    // what is left of the flat vectors: the ranges between the ones already done
    std::sort(early_ranges.begin(), early_ranges.end());
    size_t at = 0;
    for (const auto &r : early_ranges) {
        MYEA_TRY(update_range(p, at, r.first - at, early_bytes_per_param, false));
        at = r.second;
    }
    MYEA_TRY(update_range(p, at, p.n - at, early_bytes_per_param, true));
    early_ranges.clear();
    return update_finish();
}

}  // namespace myea

// =====================================================================================================================
// C ABI
// =====================================================================================================================
using myea::Net;

struct myea_hip_net { Net net; };

#define NET_OR_FAIL(n)                                             \
    do {                                                           \
        if (!(n)) { myea::set_last_error("null network handle"); return MYEA_E_INVALID; } \
    } while (0)

extern "C" {

const char *myea_hip_last_error(void) { return myea::g_last_error; }

int myea_hip_create(const myea_net_desc *desc, myea_hip_net **out)
{
    if (!desc || !out) { myea::set_last_error("myea_hip_create: null argument"); return MYEA_E_INVALID; }
    *out = nullptr;
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) { myea::set_last_error("myea_hip_create: no HIP device"); return MYEA_E_DEVICE; }
    myea_hip_net *n = new (std::nothrow) myea_hip_net();
    if (!n) return MYEA_E_NOMEM;
    const int rc = n->net.create(*desc);
    if (rc != MYEA_OK) { delete n; return rc; }
    *out = n;
    return MYEA_OK;
}

int myea_hip_destroy(myea_hip_net *n)
{
    if (!n) return MYEA_OK;
    (void)hipStreamSynchronize(n->net.stream);
    delete n;
    return MYEA_OK;
}

int myea_hip_set_stream(myea_hip_net *n, void *s) { NET_OR_FAIL(n); n->net.stream = static_cast<hipStream_t>(s); return MYEA_OK; }
int myea_hip_synchronize(myea_hip_net *n) { NET_OR_FAIL(n); MYEA_HIP_TRY(hipStreamSynchronize(n->net.stream)); return n->net.resident_check(); }

int myea_hip_set_hyper(myea_hip_net *n, const myea_hyper *h)
{
    NET_OR_FAIL(n);
    if (!h) { myea::set_last_error("set_hyper: null"); return MYEA_E_INVALID; }
    n->net.h = *h;
    // the constraint's segment table is built here so that the step itself never allocates
    if (h->regularization__max_norm_constraints != 0.f) return n->net.build_max_norm_segments();
    return MYEA_OK;
}
int myea_hip_get_hyper(myea_hip_net *n, myea_hyper *h)
{
    NET_OR_FAIL(n);
    if (!h) { myea::set_last_error("get_hyper: null"); return MYEA_E_INVALID; }
    *h = n->net.h;
    return MYEA_OK;
}
int myea_hip_set_state_propagation(myea_hip_net *n, uint32_t s)
{
    NET_OR_FAIL(n);
    if (s > MYEA_STATE_TRAINING) { myea::set_last_error("state propagation %u is not on this path", s); return MYEA_E_UNSUPPORTED; }
    if (n->net.state != s) ++n->net.mask_epoch;   // the dropout multipliers depend on the state
    n->net.state = s;
    return MYEA_OK;
}

static int copy_vec(myea_hip_net *n, float *dev, float *host_out, const float *host_in, size_t count, const char *what)
{
    if (count > n->net.d.total_parameters) { myea::set_last_error("%s: count %zu > total_parameters %llu", what, count, (unsigned long long)n->net.d.total_parameters); return MYEA_E_INVALID; }
    if (host_in) MYEA_HIP_TRY(hipMemcpyAsync(dev, host_in, count * sizeof(float), hipMemcpyHostToDevice, n->net.stream));
    else MYEA_HIP_TRY(hipMemcpyAsync(host_out, dev, count * sizeof(float), hipMemcpyDeviceToHost, n->net.stream));
    MYEA_HIP_TRY(hipStreamSynchronize(n->net.stream));
    return n->net.resident_check();
}

int myea_hip_upload_parameters(myea_hip_net *n, const float *p, size_t c)
{
    NET_OR_FAIL(n);
    if (!p) { myea::set_last_error("upload_parameters: null"); return MYEA_E_INVALID; }
    const int rc = copy_vec(n, n->net.parameters, nullptr, p, c, "upload_parameters");
    if (rc == MYEA_OK) return n->net.lstm_parameters_changed();
    return rc;
}
int myea_hip_download_parameters(myea_hip_net *n, float *p, size_t c)
{
    NET_OR_FAIL(n);
    if (!p) { myea::set_last_error("download_parameters: null"); return MYEA_E_INVALID; }
    return copy_vec(n, n->net.parameters, p, nullptr, c, "download_parameters");
}
int myea_hip_upload_optimizer_state(myea_hip_net *n, int kind, const float *p, size_t c)
{
    NET_OR_FAIL(n);
    if (kind < 0 || kind >= MYEA_STATE_KINDS || !p) { myea::set_last_error("upload_optimizer_state: bad kind %d or null", kind); return MYEA_E_INVALID; }
    return copy_vec(n, n->net.opt[kind], nullptr, p, c, "upload_optimizer_state");
}
int myea_hip_download_optimizer_state(myea_hip_net *n, int kind, float *p, size_t c)
{
    NET_OR_FAIL(n);
    if (kind < 0 || kind >= MYEA_STATE_KINDS || !p) { myea::set_last_error("download_optimizer_state: bad kind %d or null", kind); return MYEA_E_INVALID; }
    return copy_vec(n, n->net.opt[kind], p, nullptr, c, "download_optimizer_state");
}
int myea_hip_set_unit_activations(myea_hip_net *n, size_t li, const uint32_t *types, const float *steep, size_t count)
{
    NET_OR_FAIL(n);
    return n->net.set_unit_activations(li, types, steep, count);
}

int myea_hip_upload_masks(myea_hip_net *n, const uint8_t *m, size_t c)
{
    NET_OR_FAIL(n);
    if (!m || c > n->net.d.total_mask_units) { myea::set_last_error("upload_masks: null or count %zu > %llu", c, (unsigned long long)n->net.d.total_mask_units); return MYEA_E_INVALID; }
    MYEA_HIP_TRY(hipMemcpyAsync(n->net.masks, m, c, hipMemcpyHostToDevice, n->net.stream));
    MYEA_HIP_TRY(hipStreamSynchronize(n->net.stream));
    ++n->net.mask_epoch;
    return MYEA_OK;
}
int myea_hip_upload_zoneout_masks(myea_hip_net *n, const uint8_t *m, size_t c)
{
    NET_OR_FAIL(n);
    if (!m || c != n->net.zoneout_count) { myea::set_last_error("upload_zoneout_masks: null or count %zu != %zu (2 x T x cells of the LSTM layers)", c, n->net.zoneout_count); return MYEA_E_INVALID; }
    if (c == 0) return MYEA_OK;
    MYEA_HIP_TRY(hipMemcpyAsync(n->net.zoneout_masks, m, c, hipMemcpyHostToDevice, n->net.stream));
    MYEA_HIP_TRY(hipStreamSynchronize(n->net.stream));
    return MYEA_OK;
}
int myea_hip_set_dropout_seed(myea_hip_net *n, uint64_t seed)
{
    NET_OR_FAIL(n);
    n->net.dropout_seed = seed;
    n->net.dropout_stream = 0;
    return MYEA_OK;
}
int myea_hip_upload_dropout_noise(myea_hip_net *n, size_t li, const float *noise, size_t count, int on_device)
{
    NET_OR_FAIL(n);
    if (li >= n->net.d.n_layers || !n->net.L[li].noise) { myea::set_last_error("upload_dropout_noise: layer %zu has no Gaussian / Uout dropout", li); return MYEA_E_INVALID; }
    myea::DevLayer &o = n->net.L[li];
    if (!noise && count == 0) { o.noise_uploaded = false; return MYEA_OK; }   // back to the device generator
    const bool shake = n->net.d.layers[li].type_layer == MYEA_LAYER_RESIDUAL;
    const size_t TB = (size_t)n->net.d.number_recurrent_depth * n->net.d.batch_size;
    const size_t want = shake ? TB * (1 + 2 * o.NH) : TB * o.AH;
    if (!noise || count != want) { myea::set_last_error("upload_dropout_noise: null or count %zu != %zu (%s)", count, want, shake ? "T x batch_size x (1 + 2 x block width)" : "T x batch_size x activation units"); return MYEA_E_INVALID; }
    MYEA_HIP_TRY(hipMemcpyAsync(o.noise, noise, count * sizeof(float), on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, n->net.stream));
    MYEA_HIP_TRY(hipStreamSynchronize(n->net.stream));
    o.noise_uploaded = true;
    return MYEA_OK;
}
int myea_hip_clear_training_arrays(myea_hip_net *n)
{
    NET_OR_FAIL(n);
    const size_t bytes = n->net.d.total_parameters * sizeof(float);
    MYEA_HIP_TRY(hipMemsetAsync(n->net.gradient, 0, bytes, n->net.stream));
    n->net.gradient_known_zero(true);
    return n->net.clear_optimizer();
}

int myea_hip_forward_pass(myea_hip_net *n, size_t B, const float *x, int dev) { NET_OR_FAIL(n); return n->net.forward_pass(B, x, dev); }
int myea_hip_compute_error(myea_hip_net *n, size_t B, const float *y, int dev) { NET_OR_FAIL(n); return n->net.compute_error(B, y, dev); }
int myea_hip_compute_loss(myea_hip_net *n, size_t B, const float *y, int dev) { NET_OR_FAIL(n); return n->net.compute_loss(B, y, dev); }
int myea_hip_compute_accuracy_r(myea_hip_net *n, size_t B, const float *y, int dev, float mean_d, float mean_y) { NET_OR_FAIL(n); return n->net.compute_accuracy_r(B, y, dev, mean_d, mean_y); }
int myea_hip_gather_examples(myea_hip_net *n, float *dst, const float *src, size_t examples, size_t row_floats, const uint64_t *index, int index_on_device, size_t B)
{
    NET_OR_FAIL(n);
    return n->net.gather_examples(dst, src, examples, row_floats, index, index_on_device, B);
}
int myea_hip_device_buffer_create(size_t floats, const float *host, float **out)
{
    if (!out || floats == 0) { myea::set_last_error("device_buffer_create: null or empty"); return MYEA_E_INVALID; }
    *out = nullptr;
    void *q = nullptr;
    if (hipMalloc(&q, floats * sizeof(float)) != hipSuccess) { (void)hipGetLastError(); myea::set_last_error("device_buffer_create: out of device memory (%zu floats)", floats); return MYEA_E_NOMEM; }
    if (host) {
        const hipError_t e = hipMemcpy(q, host, floats * sizeof(float), hipMemcpyHostToDevice);
        if (e != hipSuccess) { (void)hipFree(q); myea::set_last_error("device_buffer_create: %s", hipGetErrorString(e)); return MYEA_E_DEVICE; }
    }
    *out = static_cast<float *>(q);
    return MYEA_OK;
}
int myea_hip_device_buffer_destroy(float *device)
{
    if (device) MYEA_HIP_TRY(hipFree(device));
    return MYEA_OK;
}
int myea_hip_backward_pass(myea_hip_net *n, size_t B) { NET_OR_FAIL(n); return n->net.backward_pass(B); }
int myea_hip_update_derivative_weight(myea_hip_net *n, size_t B, size_t first, size_t end) { NET_OR_FAIL(n); return n->net.update_derivative_weight(B, first, end); }
int myea_hip_update_derivative_weight_no_alloc(myea_hip_net *n, size_t B, size_t first, size_t end) { NET_OR_FAIL(n); return n->net.update_derivative_weight_no_alloc(B, first, end); }
int myea_hip_backward_pass_and_update_derivative_weight(myea_hip_net *n, size_t B) { NET_OR_FAIL(n); return n->net.backward_pass_and_update_derivative_weight(B); }
int myea_hip_update_parameter(myea_hip_net *n, size_t B, size_t ts) { NET_OR_FAIL(n); return n->net.update_parameter(B, ts); }
int myea_hip_backward_pass_update_derivative_weight_and_update_parameter(myea_hip_net *n, size_t B, size_t ts)
{
    NET_OR_FAIL(n);
    return n->net.backward_pass_update_derivative_weight_and_update_parameter(B, ts);
}

int myea_hip_reset_loss(myea_hip_net *n)
{
    NET_OR_FAIL(n);
    // a fill kernel, not a memset: callers may capture their step in a graph
    return myea::launch_fill(n->net.stream, reinterpret_cast<float *>(n->net.loss_acc), 8 * sizeof(double) / sizeof(float), 0.f);
}
int myea_hip_get_loss(myea_hip_net *n, myea_loss_state *s)
{
    NET_OR_FAIL(n);
    if (!s) { myea::set_last_error("get_loss: null"); return MYEA_E_INVALID; }
    double v[8];
    MYEA_HIP_TRY(hipMemcpyAsync(v, n->net.loss_acc, sizeof(v), hipMemcpyDeviceToHost, n->net.stream));
    MYEA_HIP_TRY(hipStreamSynchronize(n->net.stream));
    {
        const int rc = n->net.resident_check();
        if (rc != MYEA_OK) return rc;
    }
    s->loss_values = v[0]; s->number_loss = (uint64_t)v[1]; s->accuracy_value = v[2]; s->number_bit_fail = (uint64_t)v[3];
    for (int k = 0; k < 4; ++k) s->accuracy_r[k] = v[4 + k];
    return MYEA_OK;
}

int myea_hip_download_gradient(myea_hip_net *n, float *g, size_t c)
{
    NET_OR_FAIL(n);
    if (!g) { myea::set_last_error("download_gradient: null"); return MYEA_E_INVALID; }
    return copy_vec(n, n->net.gradient, g, nullptr, c, "download_gradient");
}
int myea_hip_upload_gradient(myea_hip_net *n, const float *g, size_t c)
{
    NET_OR_FAIL(n);
    if (!g) { myea::set_last_error("upload_gradient: null"); return MYEA_E_INVALID; }
    n->net.gradient_known_zero(false);
    return copy_vec(n, n->net.gradient, nullptr, g, c, "upload_gradient");
}

int myea_hip_download_tensor(myea_hip_net *n, size_t li, int kind, float *host, size_t count)
{
    NET_OR_FAIL(n);
    if (!host || li >= n->net.d.n_layers) { myea::set_last_error("download_tensor: null or layer %zu out of range", li); return MYEA_E_INVALID; }
    myea::DevLayer &o = n->net.L[li];
    const size_t T = n->net.d.number_recurrent_depth, full = T * n->net.d.batch_size * o.H, th = T * o.NH;
    const float *p = nullptr;
    size_t c = full;
    switch (kind) {
    case MYEA_TENSOR_OUTPUTS: p = n->net.layer_outputs(li); break;
    case MYEA_TENSOR_SUMMATIONS: p = o.summations; break;
    case MYEA_TENSOR_ERRORS: p = o.neuron_errors; break;
    case MYEA_TENSOR_NORM_HATS: p = o.hats; c = T * n->net.d.batch_size * o.NH; break;
    case MYEA_TENSOR_DROPOUT_NOISE: p = o.noise; c = n->net.d.layers[li].type_layer == MYEA_LAYER_RESIDUAL ? T * n->net.d.batch_size * (1 + 2 * o.NH) : T * n->net.d.batch_size * o.AH; break;
    case MYEA_TENSOR_INPUT_SIDE_ERRORS:
        if (o.group == 2) p = n->net.L[li - 1].neuron_errors;   // what the member handed to the one before it (an LSTM there adds its recurrent terms to it afterwards)
        else if (o.group == 1) p = o.in_errors;
        c = T * n->net.d.batch_size * o.In;
        break;
    case MYEA_TENSOR_NORM_MEANS: p = o.means; c = th; break;
    case MYEA_TENSOR_NORM_VARIANCES: p = o.variances; c = th; break;
    case MYEA_TENSOR_NORM_MEANS_AVERAGES: p = o.means_averages; c = th; break;
    case MYEA_TENSOR_NORM_VARIANCES_AVERAGES: p = o.variances_averages; c = th; break;
    default: p = n->net.lstm_tensor(li, kind, &c); break;
    }
    if (!p) { myea::set_last_error("download_tensor: layer %zu has no tensor of kind %d", li, kind); return MYEA_E_INVALID; }
    if (count > c) { myea::set_last_error("download_tensor: count %zu > tensor length %zu", count, c); return MYEA_E_INVALID; }
    MYEA_HIP_TRY(hipMemcpyAsync(host, p, count * sizeof(float), hipMemcpyDeviceToHost, n->net.stream));
    MYEA_HIP_TRY(hipStreamSynchronize(n->net.stream));
    return n->net.resident_check();
}

int myea_hip_upload_tensor(myea_hip_net *n, size_t li, int kind, const float *host, size_t count)
{
    NET_OR_FAIL(n);
    if (!host || li >= n->net.d.n_layers) { myea::set_last_error("upload_tensor: null or layer %zu out of range", li); return MYEA_E_INVALID; }
    myea::DevLayer &o = n->net.L[li];
    float *p = kind == MYEA_TENSOR_NORM_MEANS_AVERAGES ? o.means_averages : (kind == MYEA_TENSOR_NORM_VARIANCES_AVERAGES ? o.variances_averages : nullptr);
    size_t want = (size_t)n->net.d.number_recurrent_depth * o.NH;
    if (!p && o.lstm) p = n->net.lstm_norm_statistics(li, kind, &want);   // one group of a normalised LSTM layer
    if (!p) { myea::set_last_error("upload_tensor: layer %zu has no running statistics of kind %d", li, kind); return MYEA_E_INVALID; }
    if (count != want) { myea::set_last_error("upload_tensor: count %zu != %zu (T x normalised units)", count, want); return MYEA_E_INVALID; }
    MYEA_HIP_TRY(hipMemcpyAsync(p, host, count * sizeof(float), hipMemcpyHostToDevice, n->net.stream));
    MYEA_HIP_TRY(hipStreamSynchronize(n->net.stream));
    return MYEA_OK;
}

int myea_hip_profile_enable(myea_hip_net *n, int enable)
{
    NET_OR_FAIL(n);
    n->net.profiling = enable != 0;
    return MYEA_OK;
}

int myea_hip_profile_read(myea_hip_net *n, int family, uint64_t *launches, double *ms, double *work)
{
    NET_OR_FAIL(n);
    if (family < 0 || family >= myea::kProfFamilies) { myea::set_last_error("profile_read: family %d", family); return MYEA_E_INVALID; }
    MYEA_HIP_TRY(hipStreamSynchronize(n->net.stream));
    for (myea::ProfEvent &e : n->net.pending) {
        float t = 0.f;
        if (hipEventElapsedTime(&t, e.start, e.stop) == hipSuccess) {
            n->net.prof_ms[e.family] += t;
            n->net.prof_work[e.family] += e.work;
            n->net.prof_launches[e.family] += e.launches;
        }
        n->net.free_events.push_back(e);
    }
    n->net.pending.clear();
    if (launches) *launches = n->net.prof_launches[family];
    if (ms) *ms = n->net.prof_ms[family];
    if (work) *work = n->net.prof_work[family];
    n->net.prof_launches[family] = 0; n->net.prof_ms[family] = 0; n->net.prof_work[family] = 0;
    return MYEA_OK;
}

int myea_hip_optimizer_update(void *stream, const myea_hyper *h, size_t count, size_t weight_count, float gradient_scale,
                              float *parameters, float *gradient, float *state0, float *state1, float *state2)
{
    if (!h || !parameters || !gradient) { myea::set_last_error("optimizer_update: null argument"); return MYEA_E_INVALID; }
    myea::UpdateParams p{};
    p.optimizer = (int)h->type_optimizer_function;
    p.n = count; p.n_weights = weight_count;
    p.w = parameters; p.g = gradient; p.s0 = state0; p.s1 = state1; p.s2 = state2;
    p.grad_scale = gradient_scale;
    p.wd = h->regularization__weight_decay;
    const float ts = h->optimizer_time_step;
    p.lr = h->learning_rate; p.mu = h->learning_momentum;
    p.variant = h->learning_momentum != 0.f ? (h->use_Nesterov ? 2 : 1) : 0;
    p.beta1 = h->adam_beta1; p.beta2 = h->adam_beta2; p.eps = h->adam_epsilon;
    p.lr_t = h->use_adam_bias_correction ? h->adam_learning_rate * std::sqrt(1.f - std::pow(h->adam_beta2, ts)) / (1.f - std::pow(h->adam_beta1, ts)) : h->adam_learning_rate;
    p.lower = h->learning_rate_final * (1.f - 1.f / (h->learning_gamma * ts + 1.f));
    p.upper = h->learning_rate_final * (1.f + 1.f / (h->learning_gamma * ts));
    if (p.optimizer == MYEA_OPTIMIZER_IRPROP_PLUS || p.optimizer == MYEA_OPTIMIZER_IRPROP_MINUS) {   // as Net::update_prepare hands them over
        p.lr = h->rprop_increase_factor; p.mu = h->rprop_decrease_factor;
        p.lower = h->rprop_delta_min; p.upper = h->rprop_delta_max;
        p.beta1 = h->loss_rprop > h->previous_loss_rprop ? 1.f : 0.f;
        p.wd = 0.f;
    }
    return myea::launch_update(static_cast<hipStream_t>(stream), p);
}

}  // extern "C"
