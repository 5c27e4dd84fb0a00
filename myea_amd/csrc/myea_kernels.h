// myea_kernels.h — internal launch interface between the net driver and the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/myea_hip.h"

namespace myea {

// ---- error plumbing -------------------------------------------------------------------------
void set_last_error(const char *fmt, ...);
int hip_fail(hipError_t e, const char *what);

#define MYEA_HIP_TRY(expr)                                             \
    do {                                                               \
        hipError_t e__ = (expr);                                       \
        if (e__ != hipSuccess) return ::myea::hip_fail(e__, #expr);    \
    } while (0)

// ---- dense contraction ------------------------------------------------------------------------
enum GemmEpilogue : int {
    EPI_NONE = 0,        // C = acc (+ C when accumulate)
    EPI_FC_FORWARD = 1,  // C = acc + bias[n]; aux_out = AF(C) * colscale[n] when act != MYEA_AF_NONE
    EPI_FC_DERIVE = 2    // C = acc * AF'(pre[m][n], steep, val[m][n])
};

struct GemmParams {
    const float *A, *B;
    float *C;
    int M, N, K;
    long lda, ldb, ldc;
    int a_k_contiguous, b_k_contiguous;
    int accumulate;
    int c_is_zero;          // with accumulate: C is known to hold zeros, so the launch may store its product instead of adding it (same values)
    int epilogue;
    const float *bias;      // EPI_FC_FORWARD, may be null
    float *aux_out;         // EPI_FC_FORWARD, [M][ldc], may be null
    const float *colscale;  // EPI_FC_FORWARD, [N] multiplier (dropout), may be null
    const float *pre;       // EPI_FC_DERIVE, [M][ldc]
    const float *val;       // EPI_FC_DERIVE, [M][ldc]
    int act;
    float steep;
    // EPI_NONE / EPI_FC_DERIVE: addend[row * ld_addend + col] joins the product before the epilogue (the shortcut
    // gradient of a residual block arriving at the same destination); may be null
    const float *addend;
    long ld_addend;
    // When not null, column sums over each block of 32 rows, taken from the accumulators on their way out (fixed order,
    // so repeatable); the consumer sums the blocks.
    //   EPI_FC_DERIVE without `hats`: [ceil(M / 32)][N], the sums of C (the bias gradient's partial sums);
    //   EPI_FC_DERIVE with `hats` ([M][ldc], the normalised values of a batch-normalised layer): [ceil(M / 32)][2][N],
    //     the sums of C * hats and of C (what the normalisation's backward pass reduces first);
    //   EPI_FC_FORWARD: [ceil(M / 32)][2][N], the sums of C and of C * C (the batch statistics of a normalisation that follows)
    float *col_partials;
    const float *hats;
    // split-K (deterministic): slab s of the K range writes its partial product to C + s * split_k_slab; the consumer
    // sums the slabs in order.  Requires EPI_NONE and accumulate == 0.  0 / 1 = off.
    int split_k;
    long split_k_slab;
    // Two-way split along k INSIDE the launch, any epilogue: when the problem has too few tiles to give every compute unit two
    // workgroups, two workgroups share a tile, each contracting over half of k; the first to finish leaves its accumulators in
    // `pair_partials`, the second adds them to its own (half 0 + half 1: the same sum whichever finishes first) and runs the
    // epilogue.  pair_partials: at least 256 x 16384 floats (256 tiles of up to 128 x 128); pair_tickets: 2 x 256 words, zero before the first use (a launch
    // leaves them zero).  One launch at a time may use a given pair of buffers.  Null = off; the launcher decides per problem.
    float *pair_partials;
    unsigned *pair_tickets;
    // The second workgroup's wait for the first one's half is bounded by pair_polls polls (gemm_pair_polls()).  When they run out
    // it stores nothing and raises *pair_fault (device memory) and *pair_host_flag (pinned host memory), either may be null; the
    // product is then incomplete, ticket and flag words are left as they are and must be cleared before the buffers' next use.
    unsigned *pair_fault, *pair_host_flag;
    unsigned pair_polls;
};
constexpr int kGemmPairTiles = 256;   // tiles the two buffers above serve

int gemm_split_k(int M, int N, int K);
// polls a tile's second workgroup waits for the first: 2^24 (seconds), or MYEA_GEMM_PAIR_SPIN_POLLS (0: give up at once, for tests
// of that path; read at every call)
unsigned gemm_pair_polls();
// true when workgroups whose ids are equal mod 8 run on one XCD of the current device (probed by one launch per device and process)
bool device_groups_share_xcd();
// true when launch_gemm, handed pair_partials / pair_tickets, would share every 128 x 128 tile's k between two workgroups
// (at most one such tile per compute unit, a k worth halving): callers size their pair buffers by it
bool gemm_pair_k_128(int M, int N, int K);
int launch_gemm(hipStream_t stream, const GemmParams &p);
// The weight gradient delta^T X of a layer with at most 32 outputs and 32 inputs over many rows, as slabs [H][In] to be added:
// narrow_dw_slabs gives their number (0: not this kernel's shape), launch_narrow_dw writes them.
int narrow_dw_slabs(size_t H, size_t In, size_t rows);
int launch_narrow_dw(hipStream_t stream, const float *delta, const float *x, float *slabs, size_t H, size_t In, size_t rows);
// dX = delta W (`a`) and dW += delta^T X (`b`) in one launch when their shapes suit it; MYEA_OK = launched, 1 = does not
// apply (launch them one after the other), negative = error
int launch_gemm_pair(hipStream_t stream, const GemmParams &a, const GemmParams &b);
// activations the FC_FORWARD / FC_DERIVE epilogues can apply (the others run as a separate kernel)
bool gemm_can_fuse_activation(int act);

// ---- elementwise / reduction kernels ------------------------------------------------------------
// rows are the leading dimension everywhere: element (r, j) at base[r * H + j].

// out[r][j] = A[r][j + sa] + B[r][j + sb] for j in [0, wo), where an operand contributes zero outside its own width
// (wa, wb) and B may be null: the zero-padded identity shortcut (narrower operand shifted by -padding) and its gradient
// (wider operand cropped at +padding).  out may alias neither operand unless the shifts are zero.
int launch_padded_add(hipStream_t s, size_t rows, size_t wo, const float *a, size_t wa, long sa,
                      const float *b, size_t wb, long sb, float *out);
// y = AF(x) * colscale[j]  (colscale may be null); x and y may alias.
int launch_activation(hipStream_t s, int act, size_t rows, size_t H, const float *x, float *y, const float *colscale, const int *unit_act = nullptr);
// row softmax (max-subtracted) then * colscale
int launch_softmax(hipStream_t s, size_t rows, size_t H, const float *x, float *y, const float *colscale);
// dx = dy * AF'(pre, steep, val)
// unit_act / unit_steep: optional per-column arrays [H] (element i belongs to column i % H)
int launch_activation_derive(hipStream_t s, int act, float steep, size_t n, const float *pre, const float *val, const float *dy, float *dx,
                             const int *unit_act = nullptr, const float *unit_steep = nullptr, size_t H = 0);
// y[r][j] *= colscale[j]
int launch_colscale(hipStream_t s, size_t rows, size_t H, float *y, const float *colscale);
// colscale[j] = mask[j] ? on : 0   (training) over n entries
int launch_mask_to_scale(hipStream_t s, size_t n, const uint8_t *mask, float on, float *colscale);
// out[j] (+)= sum_r x[r][j]; scratch >= 64 * H floats
int launch_column_sum(hipStream_t s, size_t rows, size_t H, const float *x, float *out, int accumulate, float *scratch);
// out[col] (+)= sum over the S rows of partial[S][H], in row order
int launch_column_sum_final(hipStream_t s, size_t H, size_t S, const float *partial, float *out, int accumulate);

// batch-normalisation forward (training): statistics, running averages, r/d corrections, hats, normalizes
struct BnForwardParams {
    size_t rows, H;
    const float *x;
    const float *scale, *shift;
    float *mean, *var, *mean_avg, *var_avg, *r_corr, *d_corr;
    float *hats, *normalizes;
    float epsilon, momentum, r_max, d_max;
    int renorm;
    // optional: the activation (and the dropout column multiplier) of a layer normalised before its activation, applied
    // to the normalised value in the same pass: act_out = af(normalizes) * colscale
    float *act_out;
    const float *colscale;
    int act;
};
int launch_bn_forward_training(hipStream_t s, const BnForwardParams &p, float *scratch /* >= 128 * H floats */);
// the same from column sums the producing contraction left ([blocks][2][H]: sums of x and of x * x per block of rows): one
// launch that finishes the statistics and applies them; plain batch normalisation only (p.renorm == 0)
int launch_bn_forward_training_from_sums(hipStream_t s, const BnForwardParams &p, const float *sums, size_t blocks);
int launch_bn_forward_inference(hipStream_t s, size_t rows, size_t H, const float *x, const float *scale, const float *shift,
                                const float *mean_avg, const float *var_avg, float *normalizes);
struct BnBackwardParams {
    size_t rows, H;
    const float *x, *hats, *dy;
    const float *mean, *var, *scale, *r_corr;
    float *dscale, *dshift;  // accumulated (+=) into the gradient vector
    float *dx;
    int renorm;
};
int launch_bn_backward(hipStream_t s, const BnBackwardParams &p, float *scratch /* >= 258 * H floats */);
// the same from column sums the producing contraction left ([blocks][2][H]: sums of dy * hats and of dy per block of rows);
// plain batch normalisation only
int launch_bn_backward_from_sums(hipStream_t s, const BnBackwardParams &p, const float *sums, size_t blocks);
// every time step of a [T][Bmax][H] tensor in one launch (statistics per time step): p's tensors and per-time-step vectors are
// those of time step 0; p.rows <= Bmax rows of each time step take part.  shares: 2 * T * H floats, the scale's and the shift's
// gradient of every time step; fold_now: a second launch adds them onto p.dscale / p.dshift, otherwise the caller does that
// later (launch_bn_share_folds: the shares of many layers in one launch)
int launch_bn_forward_sequence(hipStream_t s, const BnForwardParams &p, size_t T, size_t Bmax, int training);
int launch_bn_backward_sequence(hipStream_t s, const BnBackwardParams &p, size_t T, size_t Bmax, float *shares, bool fold_now);
struct BnFoldJob { const float *shares; float *dscale, *dshift; unsigned H, T; };
// jobs: device memory; widest: the largest H among them
int launch_bn_share_folds(hipStream_t s, const BnFoldJob *jobs, size_t count, size_t widest);

// output-layer delta + loss / accuracy accumulation
struct ErrorParams {
    size_t B, T, H, Bmax;
    const float *values, *pre;   // [T][Bmax][H]
    const float *desired;        // [B][T][H]
    float *errors;               // [T][Bmax][H]
    int act;
    float steep;
    const int *unit_act;       // optional per-unit activation types [H]
    const float *unit_steep;   // optional per-unit steepnesses [H]
    int loss, accuracy;
    float accuracy_variance, bit_fail_limit;
    size_t first_t;              // number_time_delays
    int rnn_pre_quirk;           // RNN head: every unit reads the first unit's pre-activation
    double *loss_acc;            // [0]=loss sum [1]=count [2]=accuracy (R: sum desired) [3]=bit fails [4]=R: sum predicted
                                 // [5..7]=R: numerator, desired / predicted denominators
    int write_delta;             // 0 = Compute__Loss (accumulate only)
};
int launch_compute_error(hipStream_t s, const ErrorParams &p);
int launch_accuracy_r(hipStream_t s, const ErrorParams &p, float desired_mean, float predicted_mean);
int launch_gather_rows(hipStream_t s, size_t B, size_t row_floats, const unsigned long long *index, const float *src, float *dst);

// Gaussian / Uout dropout draws: noise[i] = a + b * N(0,1) (normal) or uniform in [a, b); counter-based, reproducible from
// (seed, stream_id, i)
int launch_dropout_noise(hipStream_t s, size_t n, float *noise, int normal, float a, float b, unsigned long long seed, unsigned long long stream_id);
// y *= noise (Gaussian) or y += y * noise (Uout)
int launch_dropout_noise_apply(hipStream_t s, size_t n, float *y, const float *noise, int uout);

// ShakeDrop: x[r][j] *= draws[r][j] where mask[r] is set; with a null mask x *= constant
int launch_shakedrop_apply(hipStream_t s, size_t rows, size_t W, float *x, const float *mask, const float *draws, float constant);
// x[i] = x[i] < p ? 1 : 0
int launch_threshold(hipStream_t s, size_t n, float *x, float p);

// per row of x [rows][H]: the k largest values stay, the others become 0 (ties at the cut: the lower indices stay)
int launch_k_sparse(hipStream_t s, size_t rows, size_t H, size_t k, float *x);

// Independently recurrent layer over the whole sequence: tensors are [T][Bmax][H], the first B rows of a time step in use.
struct IndRnnParams {
    size_t T, B, Bmax, H;
    const float *u;            // self weights [H]
    int act; float steep;      // layer-wide activation / steepness
    const int *unit_act;       // optional per-unit activation types [H]
    const float *unit_steep;   // optional per-unit steepnesses [H]
    const float *in;           // forward: summations or their normalisation
    float *pre_afs, *afs;      // forward: written; backward: read
    const float *colscale;     // forward: optional dropout multiplier [T][H] applied in place on the activations
    const float *dy;           // backward: delta of the layer's activations
    float *dafs;               // backward: delta of the pre-activations (the recurrence runs through it)
    float *du_rows;            // backward, optional: [B][H], the sum over t >= 1 of AF[t-1] dAF[t] of every (example, unit)
};
int launch_ind_rnn_forward(hipStream_t s, const IndRnnParams &p);
int launch_ind_rnn_backward(hipStream_t s, const IndRnnParams &p);
// du[j] += sum over t >= 1 and the batch of AF[t-1] dAF[t]; scratch: 64 * H floats
int launch_ind_rnn_self_weight_gradient(hipStream_t s, size_t T, size_t B, size_t Bmax, size_t H, const float *afs, const float *dafs, float *du, float *scratch);
int launch_clip_range(hipStream_t s, size_t n, float *w, float lo, float hi);
// the same for a table of ranges of one vector in one launch (ranges: device memory; longest: the largest count among them)
struct ClipRange { unsigned long long first; unsigned count; float lo, hi; };
int launch_clip_ranges(hipStream_t s, const ClipRange *ranges, size_t count, size_t longest, float *w);

// [B][T][W] (example rows) -> [T][Bmax][W]
int launch_scatter_time_major(hipStream_t s, size_t B, size_t T, size_t W, size_t Bmax, const float *src, float *dst);

// optimizer
int launch_sum_squares(hipStream_t s, size_t n, const float *g, float *partials /* >= 1024 */, float *out_sum);
struct UpdateParams {
    int optimizer;       // MYEA_OPTIMIZER_*
    int variant;         // GD: 0 plain, 1 momentum, 2 nesterov
    size_t n, n_weights;
    float *w, *g, *s0, *s1, *s2;
    float lr, mu, lr_t, beta1, beta2, eps, lower, upper, wd;
    const float *norm_sq;  // device scalar: sum of squares of g, or null (no clipping)
    float clip;
    float grad_scale;      // host-side multiplier (used when norm_sq is null)
    const unsigned *fault;          // device word or null: while it is not 0 the launch changes nothing
    unsigned long long *applied;    // device counter or null: incremented by a launch that found `fault` clear
};
int launch_update(hipStream_t s, const UpdateParams &p);
// every segment w[first[i] .. first[i] + len[i]) whose Euclidean norm is >= max_norm is scaled onto that norm;
// `longest` = the largest len (picks one wave or one workgroup per segment)
int launch_max_norm(hipStream_t s, size_t nseg, const unsigned long long *first, const unsigned *len, unsigned longest, float max_norm, float *w);

int launch_fill(hipStream_t s, float *p, size_t n, float v);

// ---- pooling over the feature axis (average / max), rows = (time step, example) pairs --------------------------
struct PoolParams {
    size_t rows, In, H;                       // input and output width
    unsigned kernel, stride, padding, dilation;
    int is_max;
};
// y [rows][H] <- x [rows][In]; index [rows][H] (max only): padded position of the window's first maximum
int launch_pool_forward(hipStream_t s, const PoolParams &p, const float *x, float *y, unsigned *index);
// dx [rows][In] <- dy [rows][H] (overwrites dx)
int launch_pool_backward(hipStream_t s, const PoolParams &p, const float *dy, const unsigned *index, float *dx);
// dst[0..n) += sum over the nslab slabs of n floats each, in slab order (n % 4 == 0, 16-byte aligned)
int launch_slab_sum_add(hipStream_t s, size_t n, int nslab, const float *slabs, float *dst, bool value_by_value = false);
// the same for a table of such sums in one launch (jobs: device memory; widest: the largest n among them); every sum in the
// order of the value-by-value form: four lanes a value, lane q the slabs q, q + 4, ..., the lanes' sums added in lane order
struct SlabFoldJob { const float *slabs; float *dst; unsigned n, nslab; };
int launch_slab_fold_jobs(hipStream_t s, const SlabFoldJob *jobs, size_t count, size_t widest);

// ---- fused LSTM time step (one cell per block, C % 32 == 0) ---------------------------------------------------
// all tensors are the rows of ONE time step: [B][C] (stride C) or [B][4C] gate rows z | i | f | o (stride 4C)
struct LstmFusedForward {
    size_t B, C;
    const float *h_prev;   // [B][C]   cell outputs of the step processed before this one
    const float *Wrec;     // [4C][C]  packed recurrent weights, rows z | i | f | o
    const float *bias;     // [4C]
    const float *peep;     // [3][C]   input / forget / output gate peepholes
    float *acts;           // [B][4C]  in: input sums; out: the activations z, i, f, o
    const float *c_prev;   // [B][C]
    float *c, *ca, *h;     // [B][C]   cell state, tanh(cell state), cell output
    const uint8_t *zone_state, *zone_output;   // [C] zoneout masks of this time step (1 = update), or null
};
struct LstmFusedBackward {
    size_t B, C;
    int first_step;           // the sequence's first step: no forget-gate delta
    const float *dG_next;     // [B][4C] gate deltas of the step processed after this one
    const float *WrecT;       // [C][4C] transposed packed recurrent weights
    const float *peep;        // [3][C]
    const float *acts, *acts_next;   // [B][4C]
    const float *c_prev;      // [B][C], unused on the first step
    const float *ca;          // [B][C]
    float *dh;                // [B][C]  in: delta from the layers above; out: plus the recurrent term
    float *dG;                // [B][4C] out
    float *dc;                // [B][C]  out
    const float *dc_next;     // [B][C]
};
bool lstm_fused_supported(size_t C, size_t cells_per_block);
int launch_lstm_fused_forward(hipStream_t s, const LstmFusedForward &p);
int launch_lstm_fused_backward(hipStream_t s, const LstmFusedBackward &p);
int launch_transpose(hipStream_t s, size_t rows, size_t cols, const float *src, float *dst);

// ---- LSTM time loop as one resident launch (one cell per block, C in {128, 256, 512, 1024}) --------------------------
// one direction of a layer: packed parameters and the layer's [T][Bmax][..] tensors
struct LstmResidentDir {
    const float *Wrec;     // [4C][C] packed recurrent weights, rows z | i | f | o (forward)
    const float *WrecT;    // [C][4C] their transpose (backward)
    const float *bias;     // [4C]
    const float *peep;     // [3][C]
    float *acts;           // [T][Bmax][4C] in: input sums; out: the activations z, i, f, o
    float *c, *ca, *h;     // [T][Bmax][C] cell state, tanh(cell state), cell output
    float *dh, *dG, *dc;   // backward: [T][Bmax][C] delta of the outputs (in: from above; out: plus the recurrent term), [T][Bmax][4C], [T][Bmax][C]
    float *sums;           // backward, or null: [plan.row_groups][7][C] sums over the group's examples and all time steps of
                           // dz, di, df, do (the bias gradients) and di c[step before], df c[step before], do c (the peepholes')
    const uint8_t *zone_state, *zone_output;   // zoneout masks [T][zone_stride] (1 = update) or null
    size_t zone_stride;
    int reverse;           // walks time from T - 1 down to 0
};
struct LstmResidentPlan {
    bool ok = false;       // the resident form applies
    bool agent = false;    // groups wider than one XCD: device-scope exchange
    bool backward = false; // the backward loop has a resident form too
    bool ksplit = false;   // ... and it is the one split along k, which needs the exchange buffer
    bool ksplit_available = false;   // the k form exists for this layer (a caller may set ksplit when other work shares the device)
    int cells = 0, members = 0, rs = 0, row_groups = 0, grid = 0, cus = 0;
};
int lstm_resident_plan(size_t C, size_t cells_per_block, size_t B, int dirs, LstmResidentPlan *plan);
size_t lstm_resident_sync_words();
// sync: lstm_resident_sync_words() unsigneds of device memory (cleared by the call); host_flag: a pinned host word the
// kernel sets when a bounded wait gave up (1) or the members of a group did not share an XCD (2); fault: a device word set
// to 1 on the same occasions and never cleared by these calls (null: none)
int launch_lstm_resident_forward(hipStream_t s, const LstmResidentPlan &plan, size_t T, size_t B, size_t Bmax, size_t C, int dirs,
                                 const LstmResidentDir *dir, unsigned *sync, unsigned *host_flag, unsigned *fault);
// dh must hold the delta from the layers above for every time step.  exchange: device memory of at least
// lstm_resident_exchange_floats(C, B, dirs) floats, 16-byte aligned, when plan.ksplit (its contents do not matter); else unused
size_t lstm_resident_exchange_floats(size_t C, size_t B, int dirs);
int launch_lstm_resident_backward(hipStream_t s, const LstmResidentPlan &plan, size_t T, size_t B, size_t Bmax, size_t C, int dirs,
                                  const LstmResidentDir *dir, unsigned *sync, unsigned *host_flag, unsigned *fault, float *exchange, size_t exchange_floats);

}  // namespace myea
