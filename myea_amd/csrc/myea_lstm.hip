// myea_lstm.hip — LSTM-with-peephole layers on gfx950: forward, BPTT and weight gradients.
//
// MI355X-first structure.  The reference keeps the gate weights interleaved per block inside the flat parameter
// vector (Prepare__Connections__LSTM, Neural_Network__Prepare_Connections.cpp:82-222) and walks them with scalar
// dot products per example.  Here the flat vector stays the source of truth (upload / download / optimizer run
// on it unchanged) and a packed device copy feeds the MFMA contractions:
//     Win  [G][In],  Wrec [G][C],  peep [3][C],   rows ordered  z (C cells) | i (K) | f (K) | o (K),  G = C + 3K
// refreshed by one gather kernel whenever the parameters change.  With that order the four bias vectors are one
// contiguous [G] slice of the flat vector at Layer::first_bias_connection_index, exactly where the reference reads
// them.  Per layer:
//   forward   one contraction over all time steps for the input sums  (T*B x G x In),
//             per step one contraction h[t-1] Wrec^T accumulated onto them and one fused gate kernel;
//   backward  per step one contraction dG[t+1] Wrec accumulated onto dh[t] and one fused gate-delta kernel,
//             then ONE contraction dG Win for the layer below;
//   weights   two contractions dG^T X (K = T*B) and dG[1..]^T h[..T-2] into packed scratch + scatter-add into the
//             flat gradient, a column reduction for the three peephole vectors, a column sum for the biases.
//
// NN/ = Neural_Network_Library_Windows/Source_Files/Neural_Network/.
#include <cstdlib>
#include <type_traits>

#include "myea_device_af.h"
#include "myea_kernels.h"
#include "myea_net.h"
#include "myea_reduce.h"

namespace myea {

struct LstmLayer {
    size_t K = 0, cpb = 0, C = 0, G = 0, In = 0, per_block = 0, base = 0;
    size_t bias = 0;        // flat index of the direction's bias vectors z | i | f | o
    bool reverse = false;   // second direction of a bidirectional layer: walks time from T-1 down to 0
    bool own_h = false;     // bidirectional: h / dh are the direction's own buffers; else the layer's values / neuron_errors
    float *h = nullptr, *dh = nullptr;                           // [T][Bmax][C] cell outputs and their delta
    float *Win = nullptr, *Wrec = nullptr, *peep = nullptr;      // packed parameters
    float *WrecT = nullptr; // [C][G] transposed Wrec for the fused backward step; null when the fused step is not used
    const uint8_t *zone_state = nullptr, *zone_output = nullptr;   // zoneout masks [T][zone_stride], this direction's cells from 0
    size_t zone_stride = 0;
    bool fused = false;     // one launch per time step (myea_lstm_fused.hip) instead of contraction + gate kernel
    float *gWin = nullptr, *gWrec = nullptr;                     // packed gradient scratch
    float *gWin_own = nullptr, *gWrec_own = nullptr;             // the layer's own allocations behind the two pointers above
    // the recurrent weights' contraction over all time steps, when it is one 128 x 128 tile per compute unit (1024 cells): two
    // workgroups share a tile's k and meet here (the layer's own buffers: the contractions of two layers may run beside each
    // other on two streams); pair_tickets: 2 x 256 words, zero between launches
    float *pair_partials = nullptr, *pair_tickets = nullptr;
    float *acts = nullptr;  // [T][Bmax][G]: pre-activation sums, overwritten in place by z | i | f | o
    float *c = nullptr, *ca = nullptr;                           // [T][Bmax][C] cell state and tanh(cell state)
    float *dG = nullptr;    // [T][Bmax][G] deltas dz | di | df | do
    float *dc = nullptr;    // [T][Bmax][C]
    float *part = nullptr;  // split-K slabs of the per-step recurrent contractions, 16 x [Bmax][G]
    // [ceil(Bmax / 32)][7][C]: what the resident backward loop sums of its gate deltas as it goes (bias and peephole gradients
    // per group of examples); sums_groups > 0 while they belong to the deltas in dG, of a pass over sums_batch examples
    float *sums = nullptr;
    size_t sums_groups = 0, sums_batch = 0;
    // Normalised layer (one cell per block).  The eight gate sums and the cell state pass through their own normalisation at
    // every time step (NN/Neural_Network__Forward_Pass__OpenMP.cpp:1769-2340): nine groups of normalised units, 0 block input
    // from below, 1 block input recurrent, 2 cell state, 3 / 4 input gate, 5 / 6 forget gate, 7 / 8 output gate (from below /
    // recurrent).  The sums stay packed as rows of [G] in the order z | i | f | o, separately for what comes from below and
    // what is recurrent, as do their normalised values, their x-hats and - in the backward pass - their deltas; a group is a
    // band of C columns of one of those tensors.  `acts` then holds the activations only.
    bool norm = false, renorm = false;
    size_t norm_param = 0;                   // flat index of the direction's first scale: [3 groups of C | 6 groups of K] in group order
    float *sin = nullptr, *srec = nullptr;   // [T][Bmax][G] sums from below / recurrent sums
    float *nin = nullptr, *nrec = nullptr;   // ... normalised
    float *hin = nullptr, *hrec = nullptr;   // ... their x-hats
    float *din = nullptr, *drec = nullptr;   // ... their deltas, after the backward pass through the normalisation
    float *nc = nullptr, *hc = nullptr;      // [T][Bmax][C] normalised cell state and its x-hat
    float *stats[9] = {};                    // per group 8 x [T][H]: mean, sigma, their running averages, r, d, d mean, d sigma
};

namespace {

#define MYEA_TRY(expr)                    \
    do {                                  \
        int rc__ = (expr);                \
        if (rc__ != MYEA_OK) return rc__; \
    } while (0)

constexpr size_t kMaxSlabs = 16;
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct LstmGeom {
    size_t K, cpb, C, G, In, per_block, base;
};

// flat index of packed element (row r of Win / Wrec, column a), NN/Neural_Network__Prepare_Connections.cpp:123-217
__device__ __forceinline__ size_t flat_index(const LstmGeom &g, size_t r, size_t a, bool recurrent)
{
    if (r < g.C) {
        const size_t k = r / g.cpb, j = r % g.cpb;
        return g.base + k * g.per_block + j * (g.In + g.C) + (recurrent ? g.In + a : a);
    }
    const size_t gate = (r - g.C) / g.K, k = (r - g.C) % g.K;
    const size_t gates0 = g.base + k * g.per_block + g.cpb * (g.In + g.C);
    return recurrent ? gates0 + 3 * g.In + gate * g.C + a : gates0 + gate * g.In + a;
}
__device__ __forceinline__ size_t peep_index(const LstmGeom &g, size_t gate, size_t c)
{
    const size_t k = c / g.cpb, j = c % g.cpb;
    return g.base + k * g.per_block + g.cpb * (g.In + g.C) + 3 * g.In + 3 * g.C + gate * g.cpb + j;
}

// One workgroup per packed row (the index arithmetic of the flat layout once per row, on the scalar unit; lanes walk the row's
// columns, which are consecutive in both layouts); the last workgroup takes the peepholes.
__global__ __launch_bounds__(kBlock) void lstm_gather_kernel(LstmGeom g, const float *flat, float *Win, float *Wrec, float *peep)
{
    const size_t r = blockIdx.x;
    if (r == g.G) {
        for (size_t q = threadIdx.x; q < 3 * g.C; q += kBlock) peep[q] = flat[peep_index(g, q / g.C, q % g.C)];
        return;
    }
    const float *from_in = flat + flat_index(g, r, 0, false), *from_rec = flat + flat_index(g, r, 0, true);
    float *win = Win + r * g.In, *wrec = Wrec + r * g.C;
    for (size_t a = threadIdx.x; a < g.In; a += kBlock) win[a] = from_in[a];
    for (size_t a = threadIdx.x; a < g.C; a += kBlock) wrec[a] = from_rec[a];
}

// flat gradient += packed gradient (every flat slot is owned by exactly one packed element: no atomics)
// gWin / gWrec hold s_in / s_rec split-K slabs, summed in slab order.  One workgroup per packed row, as above; a lane takes
// four consecutive columns when the widths allow (the slabs as 16-byte loads; the flat rows start at any dword).
__global__ __launch_bounds__(kBlock) void lstm_scatter_add_kernel(LstmGeom g, float *flat, const float *gWin, int s_in, const float *gWrec, int s_rec)
{
    const size_t r = blockIdx.x, n_in = g.G * g.In, n_rec = g.G * g.C;
    float *to_in = flat + flat_index(g, r, 0, false), *to_rec = flat + flat_index(g, r, 0, true);
    const float *win = gWin + r * g.In, *wrec = gWrec + r * g.C;
    if (((g.In | g.C) & 3) == 0) {
        const size_t q_in = g.In / 4, q_all = q_in + (s_rec > 0 ? g.C / 4 : 0);
        for (size_t q = threadIdx.x; q < q_all; q += kBlock) {
            const bool rec = q >= q_in;
            const size_t a = (rec ? q - q_in : q) * 4, slab = rec ? n_rec : n_in;
            const float *from = (rec ? wrec : win) + a;
            const int slabs = rec ? s_rec : s_in;
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            for (int s = 0; s < slabs; ++s) v += *reinterpret_cast<const f32x4 *>(from + (size_t)s * slab);
            float *to = (rec ? to_rec : to_in) + a;
#pragma unroll
            for (int e = 0; e < 4; ++e) to[e] += v[e];
        }
        return;
    }
    for (size_t a = threadIdx.x; a < g.In; a += kBlock) {
        float v = 0.f;
        for (int s = 0; s < s_in; ++s) v += win[(size_t)s * n_in + a];
        to_in[a] += v;
    }
    if (s_rec > 0)
        for (size_t a = threadIdx.x; a < g.C; a += kBlock) {
            float v = 0.f;
            for (int s = 0; s < s_rec; ++s) v += wrec[(size_t)s * n_rec + a];
            to_rec[a] += v;
        }
}

__device__ __forceinline__ float sigmoid_f(float s) { return 1.f / (1.f + expf(-s)); }
__device__ __forceinline__ float tanh_f(float s) { return 2.f / (1.f + expf(-2.f * s)) - 1.f; }  // AF_TANH_real

// One lane per (example, block).  Forward_Pass__LSTM__Gates_CIF_AF_State (NN/Neural_Network__Recurrent_Forward_Pass__
// OpenMP.cpp:1042-1191), __States_AF (:1547-1582), __Output (:1351-1418).  `acts` holds input + recurrent sums on
// entry (the contraction accumulated them) and the activations on exit.  First step: no forget gate, no input-gate
// peephole, c = i z; the output gate peeps at c[t].
// `part` holds `nparts` slabs [B][G] of the recurrent contraction h[t-1] Wrec^T (split along K), summed here in order.
__global__ __launch_bounds__(kBlock) void lstm_forward_step_kernel(LstmGeom g, size_t B, int first, const float *bias, const float *peep,
                                                                   float *acts, const float *c_prev, float *c, float *ca, float *h,
                                                                   const float *part, int nparts, const float *h_prev,
                                                                   const uint8_t *zone_state, const uint8_t *zone_output)
{
    const size_t n = B * g.K;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < n; idx += (size_t)gridDim.x * kBlock) {
        const size_t b = idx / g.K, k = idx % g.K;
        float *row = acts + b * g.G;
        for (int s = 0; s < nparts; ++s) {   // recurrent sums join the input sums
            const float *pr = part + ((size_t)s * B + b) * g.G;
            row[g.C + k] += pr[g.C + k];
            row[g.C + g.K + k] += pr[g.C + g.K + k];
            row[g.C + 2 * g.K + k] += pr[g.C + 2 * g.K + k];
            for (size_t j = 0; j < g.cpb; ++j) row[k * g.cpb + j] += pr[k * g.cpb + j];
        }
        const size_t cell0 = b * g.C + k * g.cpb;
        const float *pi = peep + k * g.cpb, *pf = peep + g.C + k * g.cpb, *po = peep + 2 * g.C + k * g.cpb;
        float si = row[g.C + k] + bias[g.C + k];
        float gi, gf = 0.f;
        if (!first) {
            float sf = row[g.C + g.K + k] + bias[g.C + g.K + k];
            for (size_t j = 0; j < g.cpb; ++j) { const float cp = c_prev[cell0 + j]; si += cp * pi[j]; sf += cp * pf[j]; }
            gf = sigmoid_f(sf);
        }
        gi = sigmoid_f(si);
        row[g.C + k] = gi;
        row[g.C + g.K + k] = gf;
        float so = row[g.C + 2 * g.K + k] + bias[g.C + 2 * g.K + k];
        for (size_t j = 0; j < g.cpb; ++j) {
            const size_t cc = k * g.cpb + j;
            const float z = tanh_f(row[cc] + bias[cc]);
            row[cc] = z;
            float cs = first ? z * gi : z * gi + gf * c_prev[cell0 + j];
            // zoneout of the cell state: a masked-out cell keeps its previous state, 0 on the first step
            // (Forward_Pass__LSTM__Gates_CIF_AF_State__Zoneout, NN/Neural_Network__Recurrent_Forward_Pass__Loop.cpp:1285-1288, 1331-1334)
            if (zone_state && !zone_state[cc]) cs = first ? 0.f : c_prev[cell0 + j];
            c[cell0 + j] = cs;
            ca[cell0 + j] = tanh_f(cs);
            so += cs * po[j];
        }
        const float go = sigmoid_f(so);
        row[g.C + 2 * g.K + k] = go;
        for (size_t j = 0; j < g.cpb; ++j) {
            float hv = ca[cell0 + j] * go;
            // zoneout of the cell output (Forward_Pass__LSTM__Output__Zoneout, :1475-1478, 1520-1523)
            if (zone_output && !zone_output[k * g.cpb + j]) hv = first ? 0.f : h_prev[cell0 + j];
            h[cell0 + j] = hv;
        }
    }
}

// One lane per (example, block).  Backward_Pass__LSTM_Derivative__Output (elementwise part, NN/Neural_Network__
// Recurrent_Backward_Pass__OpenMP.cpp:1228-1240), __Cell_State_AF (:1275-1327), __Gates_CIF_AF_State (:1329-1604).
// dh[t] already holds the delta from the layers above plus the recurrent term dG[t+1] Wrec.
//   mode 0: T == 1            (no gate deltas are computed: no branch of the reference matches)
//   mode 1: last step, T > 1  (only the output-gate peephole term; delta i and delta f computed)
//   mode 2: middle step       (all future terms)
//   mode 3: first step, T > 1 (all future terms; delta f is not written)
__global__ __launch_bounds__(kBlock) void lstm_backward_step_kernel(LstmGeom g, size_t B, int mode, const float *peep, const float *acts,
                                                                    const float *acts_next, const float *c_prev, const float *ca,
                                                                    float *dh, float *dG, const float *dG_next, float *dc,
                                                                    const float *dc_next, const float *part, int nparts)
{
    const size_t n = B * g.K;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < n; idx += (size_t)gridDim.x * kBlock) {
        const size_t b = idx / g.K, k = idx % g.K;
        const float *row = acts + b * g.G;
        float *drow = dG + b * g.G;
        const size_t cell0 = b * g.C + k * g.cpb;
        if (nparts > 0) {   // recurrent delta dG[t+1] Wrec (slabs along K) joins the delta from the layers above
            for (size_t j = 0; j < g.cpb; ++j) {
                float v = dh[cell0 + j];
                for (int s = 0; s < nparts; ++s) v += part[((size_t)s * B + b) * g.C + k * g.cpb + j];
                dh[cell0 + j] = v;
            }
        }
        const float gi = row[g.C + k], gf = row[g.C + g.K + k], go = row[g.C + 2 * g.K + k];
        float eo = 0.f;
        for (size_t j = 0; j < g.cpb; ++j) eo += dh[cell0 + j] * ca[cell0 + j];
        const float ddo = go * (1.f - go) * eo;
        drow[g.C + 2 * g.K + k] = ddo;
        if (mode == 0) {
            for (size_t j = 0; j < g.cpb; ++j) {
                const float a = ca[cell0 + j];
                dc[cell0 + j] = dh[cell0 + j] * go * (1.f - a * a);
                drow[k * g.cpb + j] = 0.f;
            }
            drow[g.C + k] = 0.f;
            drow[g.C + g.K + k] = 0.f;
            continue;
        }
        const bool future = mode >= 2;
        float di_n = 0.f, df_n = 0.f, f_n = 0.f;
        if (future) {
            di_n = dG_next[b * g.G + g.C + k];
            df_n = dG_next[b * g.G + g.C + g.K + k];
            f_n = acts_next[b * g.G + g.C + g.K + k];
        }
        const float *pi = peep + k * g.cpb, *pf = peep + g.C + k * g.cpb, *po = peep + 2 * g.C + k * g.cpb;
        float ei = 0.f, ef = 0.f;
        for (size_t j = 0; j < g.cpb; ++j) {
            const float a = ca[cell0 + j], z = row[k * g.cpb + j];
            float e = dh[cell0 + j] * go * (1.f - a * a);
            e += po[j] * ddo;
            if (future) {
                e += pi[j] * di_n;
                e += pf[j] * df_n;
                e += dc_next[cell0 + j] * f_n;
            }
            dc[cell0 + j] = e;
            drow[k * g.cpb + j] = e * gi * (1.f - z * z);
            ei += e * z;
            if (mode != 3) ef += e * c_prev[cell0 + j];
        }
        drow[g.C + k] = ei * (gi * (1.f - gi));
        drow[g.C + g.K + k] = mode != 3 ? ef * (gf * (1.f - gf)) : 0.f;
    }
}

// peephole gradients (NN/Neural_Network__Recurrent_Update_Derivative_Weight__OpenMP.cpp:603-625,673-683):
//   dp_i += di[t+1] c[t], dp_f += df[t+1] c[t] for t < T-1;  dp_o += do[t] c[t] for all t.
// rows of the reduction are (t, b) pairs; columns are cells.
struct PeepF {
    static constexpr int kUnroll = 1;   // four strided loads and a division per row already: more rows in flight cost registers and time
    LstmGeom g;
    size_t B, Bmax, T;
    const float *c, *dG;
    int reverse;   // the step processed after t is t - 1
    __device__ void operator()(size_t r, size_t col, double *acc) const
    {
        // (t, b) of the row in 32-bit arithmetic (the launcher holds T * B below 2^32)
        const unsigned t = (unsigned)r / (unsigned)B, b = (unsigned)r - t * (unsigned)B;
        const size_t k = col / g.cpb;
        const size_t row = (size_t)t * Bmax + b;
        const float cs = c[row * g.C + col];
        acc[2] += dG[row * g.G + g.C + 2 * g.K + k] * cs;
        if (reverse ? t > 0 : t + 1 < T) {
            const size_t nrow = (size_t)(reverse ? t - 1 : t + 1) * Bmax + b;
            acc[0] += dG[nrow * g.G + g.C + k] * cs;
            acc[1] += dG[nrow * g.G + g.C + g.K + k] * cs;
        }
    }
};

// one lane per (gate, cell): the three peephole vectors' partial sums folded in order
__global__ __launch_bounds__(kBlock) void lstm_peep_final_kernel(LstmGeom g, size_t S, const float *partial, float *flat_gradient)
{
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= 3 * g.C) return;
    const size_t gate = i / g.C, c = i % g.C;
    double s = 0.0;
#pragma unroll 8
    for (size_t y = 0; y < S; ++y) s += partial[(y * 3 + gate) * g.C + c];
    flat_gradient[peep_index(g, gate, c)] += (float)s;
}

// One cell per block: the four bias sums and the three peephole sums of a cell come from the same five values per
// (time step, example) - the cell's four gate deltas and its state - so one pass over dG and c gives all seven.  A lane
// owns one cell and walks the time steps of its examples in the direction's processing order, carrying the cell state
// of the step before (dp_i, dp_f pair the deltas of a step with the state of the step processed before it).
// grid (ceil(C / 64), S); partial[(y * 7 + v) * C + cell], v = b_z, b_i, b_f, b_o, p_i, p_f, p_o.
// A normalised layer takes the bias sums from the gates' own deltas (dG), the input and forget peepholes from the deltas of
// the gates' recurrent sums (d_rec) and the output peephole from the delta of the output gate's sum from below (d_in); a plain
// layer passes dG three times.
__global__ __launch_bounds__(kBlock) void lstm_bias_peep_partial_kernel(size_t C, size_t B, size_t Bmax, size_t T, size_t per_lane, int reverse,
                                                                        const float *__restrict__ c, const float *__restrict__ dG,
                                                                        const float *__restrict__ d_rec, const float *__restrict__ d_in, float *partial)
{
    __shared__ double red[7][4][64];
    const int cl = threadIdx.x & 63, rl = threadIdx.x >> 6;
    const size_t col = (size_t)blockIdx.x * 64 + cl, G = 4 * C;
    double acc[7];
#pragma unroll
    for (int v = 0; v < 7; ++v) acc[v] = 0.0;
    if (col < C) {
        const size_t b0 = ((size_t)blockIdx.y * 4 + rl) * per_lane, b1 = min(B, b0 + per_lane);
        for (size_t b = b0; b < b1; ++b) {
            float c_prev = 0.f;   // no step before the first: its two terms vanish
#pragma unroll 4
            for (size_t s = 0; s < T; ++s) {
                const size_t t = reverse ? T - 1 - s : s, row = t * Bmax + b;
                const float *d = dG + row * G + col;
                const float dz = d[0], di = d[C], df = d[2 * C], dout = d[3 * C], cs = c[row * C + col];
                acc[0] += dz; acc[1] += di; acc[2] += df; acc[3] += dout;
                acc[4] += d_rec[row * G + C + col] * c_prev; acc[5] += d_rec[row * G + 2 * C + col] * c_prev; acc[6] += d_in[row * G + 3 * C + col] * cs;
                c_prev = cs;
            }
        }
    }
#pragma unroll
    for (int v = 0; v < 7; ++v) red[v][rl][cl] = acc[v];
    __syncthreads();
    if (rl == 0 && col < C) {
#pragma unroll
        for (int v = 0; v < 7; ++v)
            partial[((size_t)blockIdx.y * 7 + v) * C + col] = (float)(red[v][0][cl] + red[v][1][cl] + red[v][2][cl] + red[v][3][cl]);
    }
}

// one lane per (sum, cell): partials folded in order into the bias slice (v < 4) and the peephole slots (v >= 4)
__global__ __launch_bounds__(kBlock) void lstm_bias_peep_final_kernel(LstmGeom g, size_t S, const float *partial, float *bias_gradient, float *flat_gradient)
{
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= 7 * g.C) return;
    const size_t v = i / g.C, cell = i % g.C;
    double s = 0.0;
#pragma unroll 8
    for (size_t y = 0; y < S; ++y) s += partial[(y * 7 + v) * g.C + cell];
    if (v < 4) bias_gradient[v * g.C + cell] += (float)s;
    else flat_gradient[peep_index(g, v - 4, cell)] += (float)s;
}

// column sums over (t, b) rows of a [T][Bmax][W] tensor when B < Bmax (rows are not contiguous)
struct StridedSumF {
    size_t B, Bmax, W;
    const float *x;
    __device__ void operator()(size_t r, size_t col, double *acc) const { acc[0] += x[((r / B) * Bmax + r % B) * W + col]; }
};
__global__ __launch_bounds__(kBlock) void lstm_colsum_final_kernel(size_t H, size_t S, const float *partial, float *out)
{
    const size_t col = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (col >= H) return;
    double s = 0.0;
#pragma unroll 8
    for (size_t y = 0; y < S; ++y) s += partial[y * H + col];
    out[col] += (float)s;
}

// ---- normalised layer ------------------------------------------------------------------------------------------------
// One group of normalised units at one time step: a band of H columns of row-major tensors.  Forward_Pass__Batch_
// Normalization__Training / __Batch_Renormalization__Training (NN/Neural_Network__Forward_Pass__OpenMP.cpp:4591-4837),
// __Inference (:4559-4589); backward without a shift gradient, as the LSTM path calls it
// (NN/Neural_Network__Backward_Pass__OpenMP.cpp:1469-1584, :1711-1829).
struct NormBand {
    const float *x; size_t ldx;            // what is normalised
    float *hat, *nor; size_t ldo;          // x-hat and scale * x-hat + shift
    float *d; size_t ldd;                  // backward: the delta, replaced in place
    const float *scale, *shift;
    float *dscale;                         // backward: accumulated
    float *mean, *sigma, *mean_avg, *sigma_avg, *r, *dd, *dmean, *dsigma;   // [H] of the time step
    int H;
};
constexpr int kMaxBands = 8;
struct NormBands { NormBand g[kMaxBands]; int n; };
struct NormHyper { float epsilon, momentum, r_max, d_max; int renorm; };

// grid (ceil(H / 64), bands): column sums over the batch in double, four row lanes folded in a fixed order
__global__ __launch_bounds__(kBlock) void lstm_norm_statistics_kernel(NormBands bands, size_t B, NormHyper hy)
{
    __shared__ double red[2][4][64];
    const NormBand &g = bands.g[blockIdx.y];
    const int cl = threadIdx.x & 63, rl = threadIdx.x >> 6, col = blockIdx.x * 64 + cl;
    double s1 = 0.0, s2 = 0.0;
    if (col < g.H)
        for (size_t b = rl; b < B; b += 4) { const float v = g.x[b * g.ldx + col]; s1 += v; s2 += (double)v * v; }
    red[0][rl][cl] = s1; red[1][rl][cl] = s2;
    __syncthreads();
    if (rl != 0 || col >= g.H) return;
    s1 = red[0][0][cl] + red[0][1][cl] + red[0][2][cl] + red[0][3][cl];
    s2 = red[1][0][cl] + red[1][1][cl] + red[1][2][cl] + red[1][3][cl];
    const float bscale = 1.f / (float)B;
    const float mean = (float)s1 * bscale;
    const float mavg = g.mean_avg[col] + hy.momentum * (mean - g.mean_avg[col]);
    const float sigma = sqrtf((float)s2 * bscale - mean * mean + hy.epsilon);
    const float vavg = g.sigma_avg[col] + hy.momentum * (sigma - g.sigma_avg[col]);
    g.mean[col] = mean; g.sigma[col] = sigma; g.mean_avg[col] = mavg; g.sigma_avg[col] = vavg;
    if (hy.renorm) {
        const float q = sigma / vavg, lo = 1.f / hy.r_max;
        g.r[col] = q < lo ? lo : (q > hy.r_max ? hy.r_max : q);
        const float e = (mean - mavg) / vavg;
        g.dd[col] = e < -hy.d_max ? -hy.d_max : (e > hy.d_max ? hy.d_max : e);
    }
}

// grid (x, bands); training: x-hat and the normalised value from the batch statistics; inference: from the running averages
__global__ __launch_bounds__(kBlock) void lstm_norm_apply_kernel(NormBands bands, size_t B, int training, int renorm)
{
    const NormBand &g = bands.g[blockIdx.y];
    const size_t n = B * (size_t)g.H;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        const size_t b = i / g.H, col = i % g.H;
        float v = g.x[b * g.ldx + col];
        if (!training) { g.nor[b * g.ldo + col] = g.scale[col] * ((v - g.mean_avg[col]) / g.sigma_avg[col]) + g.shift[col]; continue; }
        if (renorm) v = (v - g.mean[col]) / g.sigma[col] * g.r[col] + g.dd[col];
        else v = (v - g.mean[col]) / g.sigma[col];
        g.hat[b * g.ldo + col] = v;
        g.nor[b * g.ldo + col] = g.scale[col] * v + g.shift[col];
    }
}

// grid (ceil(H / 64), bands): the three column sums of the backward pass; the scale gradient accumulates
__global__ __launch_bounds__(kBlock) void lstm_norm_backward_sums_kernel(NormBands bands, size_t B, int renorm)
{
    __shared__ double red[3][4][64];
    const NormBand &g = bands.g[blockIdx.y];
    const int cl = threadIdx.x & 63, rl = threadIdx.x >> 6, col = blockIdx.x * 64 + cl;
    double a1 = 0.0, a2 = 0.0, a3 = 0.0;
    if (col < g.H) {
        const float vb = g.sigma[col], r = renorm ? g.r[col] : 1.f, sc = g.scale[col], mean = g.mean[col];
        const float k2 = -r / vb, k3 = -r / (vb * vb);
        for (size_t b = rl; b < B; b += 4) {
            float e = g.d[b * g.ldd + col];
            a1 += e * g.hat[b * g.ldo + col];
            e *= sc;
            a2 += e * k2;
            a3 += e * (g.x[b * g.ldx + col] - mean) * k3;
        }
    }
    red[0][rl][cl] = a1; red[1][rl][cl] = a2; red[2][rl][cl] = a3;
    __syncthreads();
    if (rl != 0 || col >= g.H) return;
    g.dscale[col] += (float)(red[0][0][cl] + red[0][1][cl] + red[0][2][cl] + red[0][3][cl]);
    g.dmean[col] = (float)(red[1][0][cl] + red[1][1][cl] + red[1][2][cl] + red[1][3][cl]);
    g.dsigma[col] = (float)(red[2][0][cl] + red[2][1][cl] + red[2][2][cl] + red[2][3][cl]);
}

__global__ __launch_bounds__(kBlock) void lstm_norm_backward_apply_kernel(NormBands bands, size_t B, int renorm)
{
    const NormBand &g = bands.g[blockIdx.y];
    const size_t n = B * (size_t)g.H;
    const float bscale = 1.f / (float)B;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        const size_t b = i / g.H, col = i % g.H;
        const float vb = g.sigma[col], r = renorm ? g.r[col] : 1.f;
        float e = g.d[b * g.ldd + col] * g.scale[col];
        e *= r / vb;
        e += g.dsigma[col] * ((g.x[b * g.ldx + col] - g.mean[col]) / ((float)B * vb));
        e += g.dmean[col] * bscale;
        g.d[b * g.ldd + col] = e;
    }
}

// One lane per (example, cell), one cell per block.  Gates_CIF_AF_State on the normalised sums
// (NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:1042-1191 with the operands of Layer::Get__Array_Summations__*__
// Activation, NN/Neural_Network.cpp:4498-4613): the recurrence and the peepholes keep the raw cell state.
__global__ __launch_bounds__(kBlock) void lstm_norm_gates_kernel(size_t C, size_t B, int first, const float *bias, const float *peep, const float *nin,
                                                                 const float *nrec, const float *c_prev, float *acts, float *c, const uint8_t *zone_state)
{
    const size_t n = B * C, G = 4 * C;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < n; idx += (size_t)gridDim.x * kBlock) {
        const size_t b = idx / C, k = idx % C;
        const float *a = nin + b * G, *r = nrec + b * G;
        float *row = acts + b * G;
        float gi, gf = 0.f, sz;
        if (!first) {
            const float cp = c_prev[b * C + k];
            float si = a[C + k] + r[C + k] + bias[C + k];
            float sf = a[2 * C + k] + r[2 * C + k] + bias[2 * C + k];
            si += cp * peep[k]; sf += cp * peep[C + k];
            gi = sigmoid_f(si); gf = sigmoid_f(sf);
            sz = a[k] + r[k] + bias[k];
        } else {
            gi = sigmoid_f(a[C + k] + bias[C + k]);
            sz = a[k] + bias[k];
        }
        const float z = tanh_f(sz);
        row[k] = z; row[C + k] = gi; row[2 * C + k] = gf;
        float cs = first ? z * gi : z * gi + gf * c_prev[b * C + k];
        if (zone_state && !zone_state[k]) cs = first ? 0.f : c_prev[b * C + k];
        c[b * C + k] = cs;
    }
}

// States_AF on the normalised cell state (:1547-1582) and Output (:1351-1418): the output gate peeps at the raw c[t]
__global__ __launch_bounds__(kBlock) void lstm_norm_output_kernel(size_t C, size_t B, int first, const float *bias, const float *peep, const float *nin,
                                                                  const float *nrec, const float *nc, const float *c, float *acts, float *ca, float *h,
                                                                  const float *h_prev, const uint8_t *zone_output)
{
    const size_t n = B * C, G = 4 * C;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < n; idx += (size_t)gridDim.x * kBlock) {
        const size_t b = idx / C, k = idx % C;
        const float a = tanh_f(nc[b * C + k]);
        ca[b * C + k] = a;
        float so = nin[b * G + 3 * C + k] + (first ? 0.f : nrec[b * G + 3 * C + k]) + bias[3 * C + k];
        so += c[b * C + k] * peep[2 * C + k];
        const float go = sigmoid_f(so);
        acts[b * G + 3 * C + k] = go;
        float hv = a * go;
        if (zone_output && !zone_output[k]) hv = first ? 0.f : h_prev[b * C + k];
        h[b * C + k] = hv;
    }
}

// Backward_Pass__LSTM_Derivative__Output (elementwise part) and __Cell_State_AF: the output gate's delta, copied to its two
// sums' deltas, and the cell state's delta through tanh (NN/Neural_Network__Recurrent_Backward_Pass__OpenMP.cpp:476-575)
__global__ __launch_bounds__(kBlock) void lstm_norm_backward_output_kernel(size_t C, size_t B, int first, const float *acts, const float *ca, float *dh,
                                                                           const float *part, int nparts, float *dG, float *din, float *drec, float *dc)
{
    const size_t n = B * C, G = 4 * C;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < n; idx += (size_t)gridDim.x * kBlock) {
        const size_t b = idx / C, k = idx % C;
        float v = dh[b * C + k];
        for (int s = 0; s < nparts; ++s) v += part[((size_t)s * B + b) * C + k];
        if (nparts > 0) dh[b * C + k] = v;
        const float go = acts[b * G + 3 * C + k], a = ca[b * C + k];
        const float ddo = (go * (1.f - go)) * (v * a);
        dG[b * G + 3 * C + k] = ddo;
        din[b * G + 3 * C + k] = ddo;
        if (!first) drec[b * G + 3 * C + k] = ddo;
        dc[b * C + k] = v * go * (1.f - a * a);
    }
}

// Backward_Pass__LSTM_Derivative__Gates_CIF_AF_State (:1329-1604) on the cell state's delta as its normalisation's backward
// pass left it, then the copies to the sums' deltas (:612-664).  compute == 0 (a single time step): no branch of the
// reference matches, the gate deltas keep their values and only the copies happen.
__global__ __launch_bounds__(kBlock) void lstm_norm_backward_gates_kernel(size_t C, size_t B, int compute, int first, int last, const float *peep,
                                                                          const float *acts, const float *acts_next, const float *c_prev, float *dG,
                                                                          const float *dG_next, float *dc, const float *dc_next, float *din, float *drec)
{
    const size_t n = B * C, G = 4 * C;
    for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < n; idx += (size_t)gridDim.x * kBlock) {
        const size_t b = idx / C, k = idx % C;
        float *drow = dG + b * G;
        if (compute) {
            const float *row = acts + b * G;
            const float z = row[k], gi = row[C + k];
            float e = dc[b * C + k];
            e += peep[2 * C + k] * drow[3 * C + k];
            if (!last) {
                e += peep[k] * dG_next[b * G + C + k];
                e += peep[C + k] * dG_next[b * G + 2 * C + k];
                e += dc_next[b * C + k] * acts_next[b * G + 2 * C + k];
            }
            dc[b * C + k] = e;
            drow[k] = e * gi * (1.f - z * z);
            drow[C + k] = (e * z) * (gi * (1.f - gi));
            if (!first) { const float gf = row[2 * C + k]; drow[2 * C + k] = (e * c_prev[b * C + k]) * (gf * (1.f - gf)); }
        }
        for (int gate = 0; gate < 3; ++gate) {
            const float v = drow[gate * C + k];
            din[b * G + gate * C + k] = v;
            if (!first) drec[b * G + gate * C + k] = v;
        }
    }
}

// ---- a normalised layer's time step in one launch -----------------------------------------------------------------------
// Everything a time step does behind its recurrent contraction touches one cell's column of a few tensors over the batch: the
// statistics are sums over the batch of that column, the gate math combines the normalised sums of the same cell.  A workgroup
// therefore owns CW cells and ALL examples, with lanes / CW row lanes: the column sums of every group meet in LDS, a wavefront
// per group finishes the statistics as lstm_norm_statistics_kernel does, and the lanes go over their rows again to apply them
// and to run the gates; a lane meets the same (example, cell) pairs in every pass, so what it wrote it may read back.
//
// What bounds such a launch is not traffic but the chain of things that wait for each other, so the kernels keep that chain short:
//  - the arguments are a few base pointers (two cache lines) and a group's tensors are computed from them; nine bands of
//    pointers would be fetched piecewise, each piece a trip to memory before the first operand can be asked for;
//  - a lane asks for its column's parameters and for its FIRST row's operands before anything waits, and keeps what it computed
//    of that row in registers for the later passes (with B <= lanes / CW no pass but the first reads a tensor);
//  - every address is a base plus one of two 32-bit offsets (rows of G = 4C floats, rows of C floats): the host keeps B * G
//    below 2^32;
//  - a column's sum over the lanes goes through the LDS unit, which all wavefronts share, as little as possible: lanes of a
//    16-lane row combine with row rotations in the vector unit, one partial per row (or per wavefront) is written, and the
//    finishing lane adds the partials in a fixed order.
// Groups: 0 z, 3 i, 5 f, 7 o from below; 1, 4, 6, 8 the recurrent sums of the same gates; 2 the cell state.
struct NormStepArgs {
    float *sum[2], *hat[2], *nor[2], *delta[2];   // [0] from below, [1] recurrent, at this time step: rows of 4C floats, z | i | f | o
    float *c, *hc, *nc, *dc;                      // the cell state's group at this time step: rows of C floats
    const float *scale, *shift;                   // of group 0; group g's at g * C
    float *dscale;
    float *stats;                                 // group 0's statistics at this time step; field f of group g at (8 g + f) * field
    unsigned cells, field;                        // C; T * C
    enum Field { kMean = 0, kSigma, kMeanAvg, kSigmaAvg, kR, kD, kDMean, kDSigma };
    __device__ __forceinline__ static int side(int g) { return (g == 0 || g == 3 || g == 5 || g == 7) ? 0 : 1; }
    __device__ __forceinline__ unsigned band(int g) const { return (unsigned)((g - 1) / 2) * cells; }   // g >= 3; 0 for groups 0 and 1
    __device__ __forceinline__ const float *x_of(int g) const { return g == 2 ? c : (g < 2 ? sum[side(g)] : sum[side(g)] + band(g)); }
    __device__ __forceinline__ float *hat_of(int g) const { return g == 2 ? hc : (g < 2 ? hat[side(g)] : hat[side(g)] + band(g)); }
    __device__ __forceinline__ float *nor_of(int g) const { return g == 2 ? nc : (g < 2 ? nor[side(g)] : nor[side(g)] + band(g)); }
    __device__ __forceinline__ float *delta_of(int g) const { return g == 2 ? dc : (g < 2 ? delta[side(g)] : delta[side(g)] + band(g)); }
    __device__ __forceinline__ float *stat(int g, int f) const { return stats + (size_t)(8 * g + f) * field; }
};
constexpr int kNormBackThreads = 512;   // the backward pass keeps more per lane: 256 registers a lane instead of 128

// st: the group's statistics at this time step, fields `field` floats apart; mean_avg_old, sigma_avg_old: the running averages as
// they stood before this step (the caller asked for them early)
__device__ __forceinline__ void norm_finish_statistics(float *st, unsigned field, unsigned col, double s1, double s2, size_t B, const NormHyper &hy, float mean_avg_old,
                                                       float sigma_avg_old, float *out)
{
    const float bscale = 1.f / (float)B;
    const float mean = (float)s1 * bscale;
    const float mavg = mean_avg_old + hy.momentum * (mean - mean_avg_old);
    const float sigma = sqrtf((float)s2 * bscale - mean * mean + hy.epsilon);
    const float vavg = sigma_avg_old + hy.momentum * (sigma - sigma_avg_old);
    st[NormStepArgs::kMean * field + col] = mean; st[NormStepArgs::kSigma * field + col] = sigma;
    st[NormStepArgs::kMeanAvg * field + col] = mavg; st[NormStepArgs::kSigmaAvg * field + col] = vavg;
    float r = 1.f, dd = 0.f;
    if (hy.renorm) {
        const float q = sigma / vavg, lo = 1.f / hy.r_max;
        r = q < lo ? lo : (q > hy.r_max ? hy.r_max : q);
        const float e = (mean - mavg) / vavg;
        dd = e < -hy.d_max ? -hy.d_max : (e > hy.d_max ? hy.d_max : e);
        st[NormStepArgs::kR * field + col] = r; st[NormStepArgs::kD * field + col] = dd;
    }
    out[0] = mean; out[1] = sigma; out[2] = r; out[3] = dd;
}

// Forward_Pass__LSTM of one time step behind the recurrent contraction (NN/Neural_Network__Forward_Pass__OpenMP.cpp:1769-2340):
// the normalisations of the gate sums, Gates_CIF_AF_State, the cell state's normalisation, States_AF and Output - the kernels
// lstm_norm_statistics / _apply / _gates / _output above in one launch.  grid: ceil(C / CW) workgroups of NT lanes.
template <bool FIRST, int CW, int NT>   // FIRST: the direction's first time step (no recurrent sums, no forget gate); CW: cells per workgroup; NT: lanes
__global__ __launch_bounds__(NT) void lstm_norm_forward_fused_kernel(NormStepArgs ns, size_t B, int training, NormHyper hy, const float *bias,
                                                                     const float *peep, const float *c_prev, float *acts, float *c, float *ca, float *h,
                                                                     const float *h_prev, const uint8_t *zone_state, const uint8_t *zone_output)
{
    constexpr int RL = NT / CW, NW = NT / 64, NP = NW * kNormPartials<CW>;
    __shared__ double red[8][2][NP][CW];
    __shared__ float st[9][4][CW];
    const int cl = threadIdx.x % CW, rl = threadIdx.x / CW, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned Cu = ns.cells, Gu = 4 * Cu, Bu = (unsigned)B, k = blockIdx.x * CW + cl;
    const bool live = k < Cu;
    const bool row0 = live && (unsigned)rl < Bu;   // the lane has a first row
    // a wavefront finishes its group's statistics with 64 / CW lanes a column; the first of them keeps the result: column fc
    const int fc = lane / (64 / CW);
    const unsigned fk = blockIdx.x * CW + fc;
    const bool finisher = lane % (64 / CW) == 0 && fk < Cu;
    const bool holder = norm_partial_holder<CW>(lane);
    const int slot = norm_partial_index<CW>(wave, lane);
    constexpr bool first = FIRST;
    constexpr int order[8] = {0, 3, FIRST ? 7 : 5, 1, 4, 6, 7, 8};
    constexpr int n = FIRST ? 3 : 8;
    static_assert(NW >= 8, "a wavefront per group finishes the statistics");
    static_assert(16 % CW == 0, "a 16-lane row holds whole batch rows");
    // offset of (row b, this lane's cell) in a tensor with rows of G floats / of C floats
    auto at_g = [&](unsigned b) { return b * Gu + k; };
    auto at_c = [&](unsigned b) { return b * Cu + k; };
    // ---- everything that does not depend on another lane
    float x0[n], scale[n], shift[n];
    float pi = 0.f, pf = 0.f, po = 0.f, bz = 0.f, bi = 0.f, bf = 0.f, bo = 0.f, csc = 0.f, csh = 0.f, cp0 = 0.f;
    float avg_mean = 0.f, avg_sigma = 0.f, avg_mean_c = 0.f, avg_sigma_c = 0.f;   // the running averages a finishing lane updates
    bool keep_state = false, keep_output = false;   // zoneout holds this cell's state / output at its previous value
#pragma unroll
    for (int i = 0; i < n; ++i) { x0[i] = 0.f; scale[i] = 0.f; shift[i] = 0.f; }
    if (row0) {
#pragma unroll
        for (int i = 0; i < n; ++i) x0[i] = ns.x_of(order[i])[at_g(rl)];
        if (!first) cp0 = c_prev[at_c(rl)];
    }
    if (live) {
        pi = peep[k]; pf = peep[Cu + k]; po = peep[2 * Cu + k];
        bz = bias[k]; bi = bias[Cu + k]; bf = bias[2 * Cu + k]; bo = bias[3 * Cu + k];
        csc = ns.scale[2 * Cu + k]; csh = ns.shift[2 * Cu + k];
#pragma unroll
        for (int i = 0; i < n; ++i) { scale[i] = ns.scale[order[i] * Cu + k]; shift[i] = ns.shift[order[i] * Cu + k]; }
        if (zone_state) keep_state = !zone_state[k];
        if (zone_output) keep_output = !zone_output[k];
    }
    if (training && finisher) {
#pragma unroll
        for (int i = 0; i < n; ++i)
            if (wave == i) { avg_mean = ns.stat(order[i], NormStepArgs::kMeanAvg)[fk]; avg_sigma = ns.stat(order[i], NormStepArgs::kSigmaAvg)[fk]; }
        if (wave == 0) { avg_mean_c = ns.stat(2, NormStepArgs::kMeanAvg)[fk]; avg_sigma_c = ns.stat(2, NormStepArgs::kSigmaAvg)[fk]; }
    }
    // ---- the statistics of the gate sums
    if (training) {
        double s1[n], s2[n];
#pragma unroll
        for (int i = 0; i < n; ++i) { s1[i] = 0.0; s2[i] = 0.0; }
        if (row0) {
#pragma unroll
            for (int i = 0; i < n; ++i) { const float v = x0[i]; s1[i] += v; s2[i] += (double)v * v; }
        }
        if (live)
            for (unsigned b = rl + RL; b < Bu; b += RL) {
#pragma unroll
                for (int i = 0; i < n; ++i) {
                    const float v = ns.x_of(order[i])[at_g(b)];
                    s1[i] += v; s2[i] += (double)v * v;
                }
            }
#pragma unroll
        for (int i = 0; i < n; ++i) {
            const double a = norm_fold_partial<CW>(s1[i]), q = norm_fold_partial<CW>(s2[i]);
            if (holder) { red[i][0][slot][cl] = a; red[i][1][slot][cl] = q; }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < n; ++i)
            if (wave == i) {
                const double a = norm_sum_partials<CW, NP>(red[i][0], lane), q = norm_sum_partials<CW, NP>(red[i][1], lane);
                if (finisher) {
                    float out[4];
                    norm_finish_statistics(ns.stat(order[i], 0), ns.field, fk, a, q, B, hy, avg_mean, avg_sigma, out);
                    st[order[i]][0][fc] = out[0]; st[order[i]][1][fc] = out[1]; st[order[i]][2][fc] = out[2]; st[order[i]][3][fc] = out[3];
                }
            }
    } else {
#pragma unroll
        for (int i = 0; i < 9; ++i)
            if (wave == i % NW && finisher) {
                st[i][0][fc] = ns.stat(i, NormStepArgs::kMeanAvg)[fk]; st[i][1][fc] = ns.stat(i, NormStepArgs::kSigmaAvg)[fk];
                st[i][2][fc] = 1.f; st[i][3][fc] = 0.f;
            }
    }
    __syncthreads();
    // ---- the normalised sums of the lane's cell, the gates, the cell state; the cell state's column sums on the way
    double c1 = 0.0, c2 = 0.0;
    float cs0 = 0.f, n7_0 = 0.f, n8_0 = 0.f;   // of the first row, for the last pass
    auto gates_row = [&](unsigned b, auto cached) {
        constexpr bool kCached = decltype(cached)::value;
        const unsigned og = at_g(b), oc = at_c(b);
        float nor[9];
#pragma unroll
        for (int i = 0; i < n; ++i) {
            const int gi = order[i];
            float v = kCached ? x0[i] : ns.x_of(gi)[og];
            v = (v - st[gi][0][cl]) / st[gi][1][cl];
            if (training) {
                if (hy.renorm) v = v * st[gi][2][cl] + st[gi][3][cl];
                ns.hat_of(gi)[og] = v;
            }
            v = scale[i] * v + shift[i];
            ns.nor_of(gi)[og] = v;
            nor[gi] = v;
        }
        float *row = acts + og;
        float gate_i, gate_f = 0.f, sz;
        const float cp = first ? 0.f : (kCached ? cp0 : c_prev[oc]);
        if (!first) {
            float si = nor[3] + nor[4] + bi;
            float sf = nor[5] + nor[6] + bf;
            si += cp * pi; sf += cp * pf;
            gate_i = sigmoid_f(si); gate_f = sigmoid_f(sf);
            sz = nor[0] + nor[1] + bz;
        } else {
            gate_i = sigmoid_f(nor[3] + bi);
            sz = nor[0] + bz;
        }
        const float z = tanh_f(sz);
        row[0] = z; row[Cu] = gate_i; row[2 * Cu] = gate_f;
        float cs = first ? z * gate_i : z * gate_i + gate_f * cp;
        if (keep_state) cs = first ? 0.f : cp;
        c[oc] = cs;
        c1 += cs; c2 += (double)cs * cs;
        if (kCached) { cs0 = cs; n7_0 = nor[7]; n8_0 = first ? 0.f : nor[8]; }
    };
    if (row0) gates_row(rl, std::true_type{});
    if (live)
        for (unsigned b = rl + RL; b < Bu; b += RL) gates_row(b, std::false_type{});
    if (training) {
        __syncthreads();   // every lane is through with red
        const double a = norm_fold_partial<CW>(c1), q = norm_fold_partial<CW>(c2);
        if (holder) { red[0][0][slot][cl] = a; red[0][1][slot][cl] = q; }
        __syncthreads();
        if (wave == 0) {
            const double sa = norm_sum_partials<CW, NP>(red[0][0], lane), sq = norm_sum_partials<CW, NP>(red[0][1], lane);
            if (finisher) {
                float out[4];
                norm_finish_statistics(ns.stat(2, 0), ns.field, fk, sa, sq, B, hy, avg_mean_c, avg_sigma_c, out);
                st[2][0][fc] = out[0]; st[2][1][fc] = out[1]; st[2][2][fc] = out[2]; st[2][3][fc] = out[3];
            }
        }
        __syncthreads();
    }
    if (!live) return;
    // ---- the cell state's normalisation, States_AF, the output gate and the cell's output
    auto output_row = [&](unsigned b, auto cached) {
        constexpr bool kCached = decltype(cached)::value;
        const unsigned og = at_g(b), oc = at_c(b);
        const float cs = kCached ? cs0 : c[oc];
        float v = (cs - st[2][0][cl]) / st[2][1][cl];
        if (training) {
            if (hy.renorm) v = v * st[2][2][cl] + st[2][3][cl];
            ns.hc[oc] = v;
        }
        v = csc * v + csh;
        ns.nc[oc] = v;
        const float a = tanh_f(v);
        ca[oc] = a;
        float so = kCached ? n7_0 + n8_0 + bo : ns.nor_of(7)[og] + (first ? 0.f : ns.nor_of(8)[og]) + bo;
        so += cs * po;
        const float go = sigmoid_f(so);
        acts[og + 3 * Cu] = go;
        float hv = a * go;
        if (keep_output) hv = first ? 0.f : h_prev[oc];
        h[oc] = hv;
    };
    if (row0) output_row(rl, std::true_type{});
    for (unsigned b = rl + RL; b < Bu; b += RL) output_row(b, std::false_type{});
}

// the three column sums of a normalisation's backward pass for one (example, cell), as lstm_norm_backward_sums_kernel forms them
struct NormBackColumn {
    float vb, r, sc, mean, k2, k3;
    __device__ __forceinline__ void load(const NormStepArgs &ns, int g, unsigned col, int renorm)
    {
        vb = ns.stat(g, NormStepArgs::kSigma)[col]; r = renorm ? ns.stat(g, NormStepArgs::kR)[col] : 1.f;
        sc = ns.scale[g * ns.cells + col]; mean = ns.stat(g, NormStepArgs::kMean)[col];
    }
    __device__ __forceinline__ void derive() { k2 = -r / vb; k3 = -r / (vb * vb); }
    // hat, x: the normalisation's forward values of this (example, cell); e: its delta
    __device__ __forceinline__ void add(float hat, float x, float e, double *a) const
    {
        a[0] += e * hat;
        e *= sc;
        a[1] += e * k2;
        a[2] += e * (x - mean) * k3;
    }
    // the last loop of the backward pass (lstm_norm_backward_apply_kernel)
    __device__ __forceinline__ float apply(float x, float d, float dmean, float dsigma, size_t B) const
    {
        float e = d * sc;
        e *= r / vb;
        e += dsigma * ((x - mean) / ((float)B * vb));
        e += dmean * (1.f / (float)B);
        return e;
    }
};

// The backward pass of one time step behind the recurrent contraction (NN/Neural_Network__Recurrent_Backward_Pass__OpenMP.cpp:476-862):
// lstm_norm_backward_output, the backward normalisations of the output gate's sums and the cell state, lstm_norm_backward_gates and
// the backward normalisations of the other gate sums in one launch.  grid: ceil(C / CW) workgroups of 8 wavefronts.
template <bool FIRST, int CW>
__global__ __launch_bounds__(kNormBackThreads) void lstm_norm_backward_fused_kernel(NormStepArgs ns, size_t B, int last, int renorm, const float *peep,
                                                                                const float *acts, const float *acts_next, const float *ca, const float *c_prev, float *dh,
                                                                                const float *part, int nparts, float *dG, const float *dG_next, float *dc,
                                                                                const float *dc_next, float *din, float *drec)
{
    constexpr int RL = kNormBackThreads / CW, NW = kNormBackThreads / 64, NP = NW * kNormPartials<CW>;
    __shared__ double red[6][3][NP][CW];
    __shared__ float fin[6][2][CW];   // dmean, dsigma of the groups in flight
    const int cl = threadIdx.x % CW, rl = threadIdx.x / CW, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned Cu = ns.cells, Gu = 4 * Cu, Bu = (unsigned)B, k = blockIdx.x * CW + cl;
    const bool live = k < Cu;
    const bool row0 = live && (unsigned)rl < Bu;
    // a wavefront finishes its group's column sums with 64 / CW lanes a column; the first of them keeps the result: column fc
    const int fc = lane / (64 / CW);
    const unsigned fk = blockIdx.x * CW + fc;
    const bool finisher = lane % (64 / CW) == 0 && fk < Cu;
    const bool holder = norm_partial_holder<CW>(lane);
    const int slot = norm_partial_index<CW>(wave, lane);
    constexpr bool first = FIRST;
    const int compute = (first && last) ? 0 : 1;
    constexpr int head[3] = {7, 2, 8};   // the output gate's sums from below, the cell state, the output gate's recurrent sums
    constexpr int nh = FIRST ? 2 : 3;
    constexpr int tail[6] = {0, 3, 5, 1, 4, 6};
    constexpr int nt = FIRST ? 2 : 6;
    constexpr int tail_gate[6] = {0, 1, 2, 0, 1, 2};   // which gate's delta a group normalises
    static_assert(NW >= 6, "a wavefront per group finishes the column sums");
    static_assert(16 % CW == 0, "a 16-lane row holds whole batch rows");
    // offset of (row b, this lane's cell) in a tensor with rows of G floats / of C floats; the cell state's group (2) has rows
    // of C floats, every other group rows of G floats
    auto at_g = [&](unsigned b) { return b * Gu + k; };
    auto at_c = [&](unsigned b) { return b * Cu + k; };
    // ---- everything that does not depend on another lane
    NormBackColumn col[nh], tc[nt];
    float p_i = 0.f, p_f = 0.f, p_o = 0.f;
    float dscale_head = 0.f, dscale_tail = 0.f;   // the scale's derivative a finishing lane adds to
    float dh0 = 0.f, go0 = 0.f, av0 = 0.f, z0 = 0.f, gi0 = 0.f, gf0 = 0.f, cp0 = 0.f, next_i0 = 0.f, next_f0 = 0.f, next_c0 = 0.f, next_gf0 = 0.f;
    float hat_head[nh], x_head[nh], hat_tail[nt], x_tail[nt], held0[3];
    constexpr int kSlabs = 16;   // at most this many partial products of the recurrent contraction (gemm_split_k's limit)
    float slab0[kSlabs];
    // the slabs of row b, asked for together: a loop that adds them one by one waits for memory once a slab
    auto load_slabs = [&](unsigned b, float *v) {
#pragma unroll
        for (int s = 0; s < kSlabs; ++s) v[s] = s < nparts ? part[((size_t)s * B + b) * Cu + k] : 0.f;
    };
#pragma unroll
    for (int s = 0; s < kSlabs; ++s) slab0[s] = 0.f;
#pragma unroll
    for (int i = 0; i < nh; ++i) { hat_head[i] = 0.f; x_head[i] = 0.f; }
#pragma unroll
    for (int i = 0; i < nt; ++i) { hat_tail[i] = 0.f; x_tail[i] = 0.f; }
    held0[0] = held0[1] = held0[2] = 0.f;
    if (row0) {
        const unsigned og = at_g(rl), oc = at_c(rl);
        dh0 = dh[oc]; go0 = acts[og + 3 * Cu]; av0 = ca[oc];
        load_slabs(rl, slab0);
#pragma unroll
        for (int i = 0; i < nh; ++i) { const unsigned o = head[i] == 2 ? oc : og; hat_head[i] = ns.hat_of(head[i])[o]; x_head[i] = ns.x_of(head[i])[o]; }
#pragma unroll
        for (int i = 0; i < nt; ++i) { hat_tail[i] = ns.hat_of(tail[i])[og]; x_tail[i] = ns.x_of(tail[i])[og]; }
        if (compute) {
            z0 = acts[og]; gi0 = acts[og + Cu];
            if (!first) { gf0 = acts[og + 2 * Cu]; cp0 = c_prev[oc]; }
            if (!last) { next_i0 = dG_next[og + Cu]; next_f0 = dG_next[og + 2 * Cu]; next_c0 = dc_next[oc]; next_gf0 = acts_next[og + 2 * Cu]; }
        } else {
#pragma unroll
            for (int gate = 0; gate < 3; ++gate) held0[gate] = dG[og + gate * Cu];
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < nh; ++i) col[i].load(ns, head[i], k, renorm);
#pragma unroll
        for (int i = 0; i < nt; ++i) tc[i].load(ns, tail[i], k, renorm);
        p_i = peep[k]; p_f = peep[Cu + k]; p_o = peep[2 * Cu + k];
    }
    if (finisher) {
#pragma unroll
        for (int i = 0; i < nh; ++i)
            if (wave == i) dscale_head = ns.dscale[head[i] * Cu + fk];
#pragma unroll
        for (int i = 0; i < nt; ++i)
            if (wave == i) dscale_tail = ns.dscale[tail[i] * Cu + fk];
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < nh; ++i) col[i].derive();
#pragma unroll
        for (int i = 0; i < nt; ++i) tc[i].derive();
    }
    // ---- the output gate's delta and the cell state's, their normalisations' sums: groups 7, 2 and, behind the first step, 8
    float ddo0 = 0.f, dcv0 = 0.f;   // of the first row, for the next pass
    {
        double a[nh][3];
#pragma unroll
        for (int i = 0; i < nh; ++i) { a[i][0] = a[i][1] = a[i][2] = 0.0; }
        auto output_row = [&](unsigned b, auto cached) {
            constexpr bool kCached = decltype(cached)::value;
            const unsigned og = at_g(b), oc = at_c(b);
            float v = kCached ? dh0 : dh[oc];
            if (kCached) {
#pragma unroll
                for (int s = 0; s < kSlabs; ++s) if (s < nparts) v += slab0[s];
            } else {
                float slab[kSlabs];
                load_slabs(b, slab);
#pragma unroll
                for (int s = 0; s < kSlabs; ++s) if (s < nparts) v += slab[s];
            }
            if (nparts > 0) dh[oc] = v;
            const float go = kCached ? go0 : acts[og + 3 * Cu], av = kCached ? av0 : ca[oc];
            const float ddo = (go * (1.f - go)) * (v * av);
            dG[og + 3 * Cu] = ddo;
            din[og + 3 * Cu] = ddo;
            if (!first) drec[og + 3 * Cu] = ddo;
            const float dcv = v * go * (1.f - av * av);
            dc[oc] = dcv;
#pragma unroll
            for (int i = 0; i < nh; ++i) {
                const unsigned o = head[i] == 2 ? oc : og;
                const float hat = kCached ? hat_head[i] : ns.hat_of(head[i])[o], x = kCached ? x_head[i] : ns.x_of(head[i])[o];
                col[i].add(hat, x, i == 1 ? dcv : ddo, a[i]);
            }
            if (kCached) { ddo0 = ddo; dcv0 = dcv; }
        };
        if (row0) output_row(rl, std::true_type{});
        if (live)
            for (unsigned b = rl + RL; b < Bu; b += RL) output_row(b, std::false_type{});
#pragma unroll
        for (int i = 0; i < nh; ++i)
#pragma unroll
            for (int v = 0; v < 3; ++v) {
                const double f = norm_fold_partial<CW>(a[i][v]);
                if (holder) red[i][v][slot][cl] = f;
            }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < nh; ++i)
        if (wave == i) {
            const double q0 = norm_sum_partials<CW, NP>(red[i][0], lane), q1 = norm_sum_partials<CW, NP>(red[i][1], lane), q2 = norm_sum_partials<CW, NP>(red[i][2], lane);
            if (finisher) {
                ns.dscale[head[i] * Cu + fk] = dscale_head + (float)q0;
                ns.stat(head[i], NormStepArgs::kDMean)[fk] = (float)q1; ns.stat(head[i], NormStepArgs::kDSigma)[fk] = (float)q2;
                fin[i][0][fc] = (float)q1; fin[i][1][fc] = (float)q2;
            }
        }
    __syncthreads();
    // ---- those normalisations' last loop, the gates' deltas, the sums of the other groups: 0, 3 and, behind the first step, 5, 1, 4, 6
    float dmean_head[nh], dsigma_head[nh];
#pragma unroll
    for (int i = 0; i < nh; ++i) { dmean_head[i] = fin[i][0][cl]; dsigma_head[i] = fin[i][1][cl]; }
    float gd0[3] = {0.f, 0.f, 0.f};   // the first row's gate deltas, for the last pass
    {
        double a[nt][3];
#pragma unroll
        for (int i = 0; i < nt; ++i) { a[i][0] = a[i][1] = a[i][2] = 0.0; }
        auto gates_row = [&](unsigned b, auto cached) {
            constexpr bool kCached = decltype(cached)::value;
            const unsigned og = at_g(b), oc = at_c(b);
            const float ddo = kCached ? ddo0 : dG[og + 3 * Cu];
            din[og + 3 * Cu] = col[0].apply(kCached ? x_head[0] : ns.x_of(7)[og], ddo, dmean_head[0], dsigma_head[0], B);
            if (!first) drec[og + 3 * Cu] = col[nh - 1].apply(kCached ? x_head[nh - 1] : ns.x_of(8)[og], ddo, dmean_head[nh - 1], dsigma_head[nh - 1], B);
            float e = col[1].apply(kCached ? x_head[1] : ns.c[oc], kCached ? dcv0 : dc[oc], dmean_head[1], dsigma_head[1], B);
            float *drow = dG + og;
            float gd[3];
            if (compute) {
                const float *row = acts + og;
                const float z = kCached ? z0 : row[0], gi = kCached ? gi0 : row[Cu];
                e += p_o * ddo;
                if (!last) {
                    e += p_i * (kCached ? next_i0 : dG_next[og + Cu]);
                    e += p_f * (kCached ? next_f0 : dG_next[og + 2 * Cu]);
                    e += (kCached ? next_c0 : dc_next[oc]) * (kCached ? next_gf0 : acts_next[og + 2 * Cu]);
                }
                dc[oc] = e;
                gd[0] = e * gi * (1.f - z * z);
                gd[1] = (e * z) * (gi * (1.f - gi));
                drow[0] = gd[0]; drow[Cu] = gd[1];
                if (!first) {
                    const float gf = kCached ? gf0 : row[2 * Cu];
                    gd[2] = (e * (kCached ? cp0 : c_prev[oc])) * (gf * (1.f - gf));
                    drow[2 * Cu] = gd[2];
                } else {
                    gd[2] = drow[2 * Cu];   // the first step has no forget gate: its delta keeps its value
                }
            } else {
                dc[oc] = e;
#pragma unroll
                for (int gate = 0; gate < 3; ++gate) gd[gate] = kCached ? held0[gate] : drow[gate * Cu];
            }
#pragma unroll
            for (int gate = 0; gate < 3; ++gate) {
                din[og + gate * Cu] = gd[gate];
                if (!first) drec[og + gate * Cu] = gd[gate];
            }
#pragma unroll
            for (int i = 0; i < nt; ++i) {
                const float hat = kCached ? hat_tail[i] : ns.hat_of(tail[i])[og], x = kCached ? x_tail[i] : ns.x_of(tail[i])[og];
                tc[i].add(hat, x, gd[tail_gate[i]], a[i]);
            }
            if (kCached) { gd0[0] = gd[0]; gd0[1] = gd[1]; gd0[2] = gd[2]; }
        };
        if (row0) gates_row(rl, std::true_type{});
        if (live)
            for (unsigned b = rl + RL; b < Bu; b += RL) gates_row(b, std::false_type{});
        __syncthreads();   // fin and red are free again
#pragma unroll
        for (int i = 0; i < nt; ++i)
#pragma unroll
            for (int v = 0; v < 3; ++v) {
                const double f = norm_fold_partial<CW>(a[i][v]);
                if (holder) red[i][v][slot][cl] = f;
            }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < nt; ++i)
        if (wave == i) {
            const double q0 = norm_sum_partials<CW, NP>(red[i][0], lane), q1 = norm_sum_partials<CW, NP>(red[i][1], lane), q2 = norm_sum_partials<CW, NP>(red[i][2], lane);
            if (finisher) {
                ns.dscale[tail[i] * Cu + fk] = dscale_tail + (float)q0;
                ns.stat(tail[i], NormStepArgs::kDMean)[fk] = (float)q1; ns.stat(tail[i], NormStepArgs::kDSigma)[fk] = (float)q2;
                fin[i][0][fc] = (float)q1; fin[i][1][fc] = (float)q2;
            }
        }
    __syncthreads();
    if (!live) return;
    // ---- the last loop of the other groups' normalisations, on the deltas this lane left in din and drec
    auto apply_row = [&](unsigned b, auto cached) {
        constexpr bool kCached = decltype(cached)::value;
        const unsigned og = at_g(b);
#pragma unroll
        for (int i = 0; i < nt; ++i) {
            float *d = ns.delta_of(tail[i]) + og;
            *d = tc[i].apply(kCached ? x_tail[i] : ns.x_of(tail[i])[og], kCached ? gd0[tail_gate[i]] : *d, fin[i][0][cl], fin[i][1][cl], B);
        }
    };
    if (row0) apply_row(rl, std::true_type{});
    for (unsigned b = rl + RL; b < Bu; b += RL) apply_row(b, std::false_type{});
}

int dev_alloc_zero(float **p, size_t count)
{
    void *q = nullptr;
    const size_t bytes = (count ? count : 1) * sizeof(float);
    hipError_t e = hipMalloc(&q, bytes);
    if (e != hipSuccess) { hip_fail(e, "hipMalloc"); return MYEA_E_NOMEM; }
    e = hipMemset(q, 0, bytes);
    if (e != hipSuccess) return hip_fail(e, "hipMemset");
    *p = static_cast<float *>(q);
    return MYEA_OK;
}

LstmGeom geom_of(const LstmLayer &q) { return LstmGeom{q.K, q.cpb, q.C, q.G, q.In, q.per_block, q.base}; }

// MYEA_LSTM_FUSED=0 in the environment keeps every layer on the generic path (contraction + gate kernel per step)
bool fused_lstm_disabled()
{
    const char *e = std::getenv("MYEA_LSTM_FUSED");
    return e && e[0] == '0';
}

// MYEA_LSTM_NORM_FUSED=0 keeps a normalised layer's time step as the sequence of statistics / apply / gate launches (read at
// every call: a test runs both forms in one process)
// The one-launch kernels address with 32-bit offsets into a time step's tensors and into a statistics field over all time
// steps: rows * (4 * cells) and steps * cells have to stay below 2^32.
bool lstm_norm_fused_allowed(size_t rows, size_t cells, size_t steps)
{
    const char *e = std::getenv("MYEA_LSTM_NORM_FUSED");
    return !(e && e[0] == '0') && rows * 4 * cells < ((size_t)1 << 32) && steps * cells < ((size_t)1 << 32);
}

// MYEA_SIDE_STREAM=0 keeps every launch on the caller's stream (for A/B timing)
bool side_stream_disabled()
{
    const char *e = std::getenv("MYEA_SIDE_STREAM");
    return e && e[0] == '0';
}

}  // namespace

int Net::lstm_create_layer(size_t li)
{
    const myea_layer_desc &l = d.layers[li];
    DevLayer &o = L[li];
    // with more cells per block the reference's indices [3] .. [8] into the layer's normalised units (NN/Neural_Network.cpp:4498-4613)
    // land on the second cell's units, not on the block's (they are laid out per block, NN/Neural_Network__Ordered.cpp:937-966)
    if (layer_uses_norm(l) && l.n_cells_per_block != 1) { set_last_error("layer %zu: a normalised LSTM layer needs one cell per block", li); return MYEA_E_UNSUPPORTED; }
    if (l.type_dropout != MYEA_DROPOUT_NONE && l.type_dropout != MYEA_DROPOUT_ZONEOUT) { set_last_error("layer %zu: dropout type %u on an LSTM layer is not on this path", li, l.type_dropout); return MYEA_E_UNSUPPORTED; }
    if (l.n_cells_per_block == 0) { set_last_error("layer %zu: LSTM needs at least one cell per block", li); return MYEA_E_INVALID; }
    const size_t T = d.number_recurrent_depth, B = d.batch_size;
    const size_t dirs = l.use_bidirectional ? 2 : 1;
    MYEA_TRY(dev_alloc_zero(&o.neuron_errors, T * B * (size_t)l.n_units * l.n_cells_per_block));  // delta of the layer's output (ptr_delta_cell_output)
    // Two directions (contract of this library: the reference overlays its two directions' buffers and has no behaviour to
    // follow): direction 1 owns the second half of the layer's blocks and the second [G] slice of its biases and walks time
    // backwards; the layer's output is the sum of both cell outputs and both receive the same delta from above.
    for (size_t dir = 0; dir < dirs; ++dir) {
        LstmLayer *q = new LstmLayer();
        (dir ? o.lstm2 : o.lstm) = q;
        q->K = l.n_units; q->cpb = l.n_cells_per_block; q->C = q->K * q->cpb; q->G = q->C + 3 * q->K; q->In = L[li].In;
        q->per_block = q->cpb * (q->In + q->C) + 3 * q->In + 3 * q->C + 3 * q->cpb;
        q->base = l.first_connection_index + dir * q->K * q->per_block;
        q->bias = l.first_bias_connection_index + dir * q->G;
        q->reverse = dir == 1;
        q->own_h = dirs == 2;
        if (l.type_dropout == MYEA_DROPOUT_ZONEOUT) {
            // ptr_array_cell_units_mask_dropout_zoneout (Reset__Parameters__Cell_Unit__Mask_Dropout, NN/Neural_Network.cpp:3964-3995):
            // per LSTM layer [T][cells of the layer], cell-state masks first, cell-output masks T x (all cells) further on
            size_t before = 0;
            for (size_t lj = 1; lj < li; ++lj)
                if (d.layers[lj].type_layer == MYEA_LAYER_LSTM) before += (size_t)d.layers[lj].n_units * d.layers[lj].n_cells_per_block * (d.layers[lj].use_bidirectional ? 2 : 1);
            q->zone_stride = q->C * dirs;
            q->zone_state = zoneout_masks + T * before + dir * q->C;
            q->zone_output = q->zone_state + zoneout_count / 2;
        }
        if (q->base + q->K * q->per_block > d.total_weights) { set_last_error("layer %zu: LSTM weight slice leaves the weight region", li); return MYEA_E_INVALID; }
        // The four bias vectors are read at bias + [0, G).  With the index as Prepare__Bias__LSTM leaves it (one direction)
        // they reach C entries into the following layers' bias slots; beyond the bias region the reference would read and
        // write outside its parameter array, which is refused here.
        if (q->bias < d.total_weights || q->bias + q->G > d.total_weights + d.total_bias) {
            set_last_error("layer %zu: LSTM bias slice [%zu, +%zu) leaves the bias region", li, q->bias, q->G);
            return MYEA_E_INVALID;
        }
        MYEA_TRY(dev_alloc_zero(&q->Win, q->G * q->In));
        MYEA_TRY(dev_alloc_zero(&q->Wrec, q->G * q->C));
        MYEA_TRY(dev_alloc_zero(&q->peep, 3 * q->C));
        q->norm = layer_uses_norm(l);
        q->renorm = l.type_normalization == MYEA_NORMALIZATION_BATCH_RENORMALIZATION;
        q->fused = !q->norm && lstm_fused_supported(q->C, q->cpb) && !fused_lstm_disabled();
        if (q->fused) MYEA_TRY(dev_alloc_zero(&q->WrecT, q->C * q->G));
        if (q->fused) MYEA_TRY(dev_alloc_zero(&q->sums, (B + 31) / 32 * 7 * q->C));
        MYEA_TRY(dev_alloc_zero(&q->gWin, kMaxSlabs * q->G * q->In));   // split-K slabs of the weight-gradient contractions
        MYEA_TRY(dev_alloc_zero(&q->gWrec, kMaxSlabs * q->G * q->C));
        q->gWin_own = q->gWin; q->gWrec_own = q->gWrec;
        if (T > 1 && gemm_pair_k_128((int)q->G, (int)q->C, (int)((T - 1) * B))) {
            MYEA_TRY(dev_alloc_zero(&q->pair_partials, (size_t)kGemmPairTiles * 128 * 128));
            MYEA_TRY(dev_alloc_zero(&q->pair_tickets, 2 * kGemmPairTiles));
        }
        MYEA_TRY(dev_alloc_zero(&q->acts, T * B * q->G));
        MYEA_TRY(dev_alloc_zero(&q->c, T * B * q->C));
        MYEA_TRY(dev_alloc_zero(&q->ca, T * B * q->C));
        MYEA_TRY(dev_alloc_zero(&q->dG, T * B * q->G));
        MYEA_TRY(dev_alloc_zero(&q->dc, T * B * q->C));
        MYEA_TRY(dev_alloc_zero(&q->part, 16 * B * q->G));
        if (q->own_h) {
            MYEA_TRY(dev_alloc_zero(&q->h, T * B * q->C));
            MYEA_TRY(dev_alloc_zero(&q->dh, T * B * q->C));
        } else { q->h = o.values; q->dh = o.neuron_errors; }
        if (q->norm) {
            q->norm_param = d.total_weights + d.total_bias + l.first_normalized_unit_index + dir * (3 * q->C + 6 * q->K);
            if (l.first_normalized_unit_index + dirs * (3 * q->C + 6 * q->K) > d.total_normalized_units) { set_last_error("layer %zu: scale/shift slice leaves its region", li); return MYEA_E_INVALID; }
            for (float **p : {&q->sin, &q->srec, &q->nin, &q->nrec, &q->hin, &q->hrec, &q->din, &q->drec}) MYEA_TRY(dev_alloc_zero(p, T * B * q->G));
            for (float **p : {&q->nc, &q->hc}) MYEA_TRY(dev_alloc_zero(p, T * B * q->C));
            MYEA_TRY(dev_alloc_zero(&q->stats[0], 9 * 8 * T * q->C));   // one block: the one-launch kernels reach every group from the first
            for (int g = 0; g < 9; ++g) {
                q->stats[g] = q->stats[0] + (size_t)g * 8 * T * q->C;
                MYEA_TRY(launch_fill(0, q->stats[g] + 3 * T * q->C, T * q->C, 1.f));   // running sigma starts at 1, NN/Neural_Network__Allocate.cpp:2612-2615
            }
            MYEA_HIP_TRY(hipDeviceSynchronize());
        }
    }
    // the widest layer sizes the buffer the members of a resident backward loop hand each other partial sums through
    if (o.lstm->fused && o.lstm->cpb == 1)
        resident_exchange_floats = std::max(resident_exchange_floats, lstm_resident_exchange_floats(o.lstm->C, B, (int)dirs));
    return MYEA_OK;
}

void Net::lstm_destroy_layer(DevLayer &o)
{
    for (LstmLayer **slot : {&o.lstm, &o.lstm2}) {
        LstmLayer *q = *slot;
        if (!q) continue;
        float *all[] = {q->Win, q->Wrec, q->WrecT, q->peep, q->gWin_own, q->gWrec_own, q->acts, q->c, q->ca, q->dG, q->dc, q->part, q->sums, q->pair_partials, q->pair_tickets, q->own_h ? q->h : nullptr, q->own_h ? q->dh : nullptr,
                        q->sin, q->srec, q->nin, q->nrec, q->hin, q->hrec, q->din, q->drec, q->nc, q->hc};
        for (float *p : all) if (p) (void)hipFree(p);
        if (q->stats[0]) (void)hipFree(q->stats[0]);   // the nine groups share one block
        delete q;
        *slot = nullptr;
    }
}

size_t Net::lstm_scratch_floats() const
{
    size_t need = 0;
    for (const DevLayer &o : L)
        if (o.lstm) { const size_t n = 64 * 3 * o.lstm->C + 64 * o.lstm->G; if (n > need) need = n; }
    return need;
}

static size_t round_up_64(size_t n) { return (n + 63) / 64 * 64; }

size_t Net::lstm_gradient_slab_floats() const
{
    size_t need = 0;
    for (const DevLayer &o : L)
        for (const LstmLayer *q : {o.lstm, o.lstm2})
            if (q) need += round_up_64(kMaxSlabs * q->G * q->In) + round_up_64(kMaxSlabs * q->G * q->C);
    return need;
}

void Net::lstm_bind_gradient_slabs(float *base)
{
    for (DevLayer &o : L)
        for (LstmLayer *q : {o.lstm, o.lstm2}) {
            if (!q) continue;
            if (!base) { q->gWin = q->gWin_own; q->gWrec = q->gWrec_own; continue; }
            q->gWin = base; base += round_up_64(kMaxSlabs * q->G * q->In);
            q->gWrec = base; base += round_up_64(kMaxSlabs * q->G * q->C);
        }
}

int Net::lstm_pair_words_clear()
{
    for (size_t li = 1; li < L.size(); ++li)
        for (LstmLayer *q : {L[li].lstm, L[li].lstm2})
            if (q && q->pair_tickets) MYEA_HIP_TRY(hipMemset(q->pair_tickets, 0, 2 * kGemmPairTiles * sizeof(unsigned)));
    return MYEA_OK;
}

// packed copies <- flat vector; called after every parameter upload and every optimizer update
int Net::lstm_parameters_changed()
{
    for (size_t li = 1; li < L.size(); ++li) {
        for (LstmLayer *q : {L[li].lstm, L[li].lstm2}) {
            if (!q) continue;
            hipLaunchKernelGGL(lstm_gather_kernel, dim3((unsigned)q->G + 1u), dim3(kBlock), 0, stream, geom_of(*q), parameters, q->Win, q->Wrec, q->peep);
            MYEA_HIP_TRY(hipGetLastError());
            if (q->WrecT) MYEA_TRY(launch_transpose(stream, q->G, q->C, q->Wrec, q->WrecT));
        }
    }
    return MYEA_OK;
}

// Recurrent__Forward_Pass__LSTM (NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:448-471): time ascending, or
// descending for the second direction (the "previous" step is then t + 1, :456-461).
// Input sums of every time step in one contraction when the rows are contiguous.
int Net::lstm_forward_inputs(size_t li, LstmLayer &q, size_t B)
{
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size;
    const float *x = layer_outputs(L[li].prev);
    const bool per_t = T > 1 && B != Bmax;
    const size_t chunks = per_t ? T : 1, rows = per_t ? B : T * B;
    for (size_t c = 0; c < chunks; ++c) {
        GemmParams g{};
        g.A = x + c * Bmax * q.In; g.lda = (long)q.In; g.a_k_contiguous = 1;
        g.B = q.Win; g.ldb = (long)q.In; g.b_k_contiguous = 1;
        g.C = (q.norm ? q.sin : q.acts) + c * Bmax * q.G; g.ldc = (long)q.G;
        g.M = (int)rows; g.N = (int)q.G; g.K = (int)q.In;
        prof_begin(0);
        MYEA_TRY(launch_gemm(stream, g));
        prof_end(2.0 * (double)rows * (double)q.G * (double)q.In);
    }
    return MYEA_OK;
}

// the s-th time step the direction processes
int Net::lstm_forward_step(LstmLayer &q, size_t B, size_t s)
{
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size;
    const float *bias = parameters + q.bias;
    const size_t t = q.reverse ? T - 1 - s : s, tp = q.reverse ? t + 1 : t - 1;  // tp: the step processed before t
    float *acts_t = q.acts + t * Bmax * q.G;
    // zoneout acts strictly in the training state (NN/Neural_Network__Forward_Pass__Loop.cpp:2088-2092)
    const bool zone = q.zone_state != nullptr && state == MYEA_STATE_TRAINING;
    const uint8_t *zs = zone ? q.zone_state + t * q.zone_stride : nullptr, *zo = zone ? q.zone_output + t * q.zone_stride : nullptr;
    int nparts = 0;
    if (s > 0 && q.fused) {   // recurrent contraction and gate math of the step in one launch
        LstmFusedForward f{};
        f.B = B; f.C = q.C;
        f.h_prev = q.h + tp * Bmax * q.C; f.Wrec = q.Wrec; f.bias = bias; f.peep = q.peep;
        f.acts = acts_t; f.c_prev = q.c + tp * Bmax * q.C;
        f.c = q.c + t * Bmax * q.C; f.ca = q.ca + t * Bmax * q.C; f.h = q.h + t * Bmax * q.C;
        f.zone_state = zs; f.zone_output = zo;
        return launch_lstm_fused_forward(stream, f);
    }
    if (s > 0) {
        GemmParams g{};
        g.A = q.h + tp * Bmax * q.C; g.lda = (long)q.C; g.a_k_contiguous = 1;
        g.B = q.Wrec; g.ldb = (long)q.C; g.b_k_contiguous = 1;
        g.C = q.part; g.ldc = (long)q.G;
        g.M = (int)B; g.N = (int)q.G; g.K = (int)q.C;
        nparts = gemm_split_k(g.M, g.N, g.K);
        g.split_k = nparts; g.split_k_slab = (long)(B * q.G);
        MYEA_TRY(launch_gemm(stream, g));
    }
    hipLaunchKernelGGL(lstm_forward_step_kernel, dim3(grid_for(B * q.K, kBlock, 8192)), dim3(kBlock), 0, stream, geom_of(q), B, (int)(s == 0), bias, q.peep,
                       acts_t, s ? q.c + tp * Bmax * q.C : nullptr, q.c + t * Bmax * q.C, q.ca + t * Bmax * q.C, q.h + t * Bmax * q.C,
                       q.part, nparts, s ? q.h + tp * Bmax * q.C : nullptr, zs, zo);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// the band of group `g` (0 .. 8) of a normalised layer at time step t
static NormBand norm_band(const LstmLayer &q, float *parameters, float *gradient, size_t total_norm, int g, size_t t, size_t T, size_t Bmax)
{
    NormBand b{};
    const size_t C = q.C, G = q.G, rows = t * Bmax;
    const bool below = g == 0 || g == 3 || g == 5 || g == 7;
    const size_t col = g == 2 ? 0 : (g < 2 ? 0 : (size_t)((g - 1) / 2) * C);   // z | i | f | o bands of the packed rows
    if (g == 2) {
        b.x = q.c + rows * C; b.ldx = C; b.hat = q.hc + rows * C; b.nor = q.nc + rows * C; b.ldo = C; b.d = q.dc + rows * C; b.ldd = C;
    } else {
        b.x = (below ? q.sin : q.srec) + rows * G + col; b.ldx = G;
        b.hat = (below ? q.hin : q.hrec) + rows * G + col; b.nor = (below ? q.nin : q.nrec) + rows * G + col; b.ldo = G;
        b.d = (below ? q.din : q.drec) + rows * G + col; b.ldd = G;
    }
    const size_t at = q.norm_param + (g < 3 ? (size_t)g * C : 3 * C + (size_t)(g - 3) * q.K);
    b.scale = parameters + at; b.shift = parameters + at + total_norm; b.dscale = gradient + at;
    float *st = q.stats[g] + t * C;
    const size_t TH = T * C;
    b.mean = st; b.sigma = st + TH; b.mean_avg = st + 2 * TH; b.sigma_avg = st + 3 * TH; b.r = st + 4 * TH; b.dd = st + 5 * TH; b.dmean = st + 6 * TH; b.dsigma = st + 7 * TH;
    b.H = (int)C;
    return b;
}

// the tensors of a normalised layer at time step t, for the one-launch kernels
static NormStepArgs norm_step_args(const LstmLayer &q, float *parameters, float *gradient, size_t total_norm, size_t t, size_t T, size_t Bmax)
{
    NormStepArgs a{};
    const size_t rg = t * Bmax * q.G, rc = t * Bmax * q.C;
    a.sum[0] = q.sin + rg; a.sum[1] = q.srec + rg; a.hat[0] = q.hin + rg; a.hat[1] = q.hrec + rg;
    a.nor[0] = q.nin + rg; a.nor[1] = q.nrec + rg; a.delta[0] = q.din + rg; a.delta[1] = q.drec + rg;
    a.c = q.c + rc; a.hc = q.hc + rc; a.nc = q.nc + rc; a.dc = q.dc + rc;
    a.scale = parameters + q.norm_param; a.shift = a.scale + total_norm; a.dscale = gradient + q.norm_param;
    a.stats = q.stats[0] + t * q.C;   // the groups' statistics are one block, 8 fields of [T][C] a group
    a.cells = (unsigned)q.C; a.field = (unsigned)(T * q.C);
    return a;
}

int Net::lstm_norm_forward_groups(LstmLayer &q, size_t B, size_t t, std::initializer_list<int> groups)
{
    NormBands bands{};
    for (int g : groups) bands.g[bands.n++] = norm_band(q, parameters, gradient, d.total_normalized_units, g, t, d.number_recurrent_depth, d.batch_size);
    if (bands.n == 0 || B == 0) return MYEA_OK;
    const bool training = state >= MYEA_STATE_TRAINING;
    const NormHyper hy{h.normalization_epsilon, h.normalization_momentum_average, h.batch_renormalization_r_correction_maximum,
                       h.batch_renormalization_d_correction_maximum, q.renorm ? 1 : 0};
    prof_begin(kProfNormalization);
    if (training) {
        hipLaunchKernelGGL(lstm_norm_statistics_kernel, dim3((unsigned)((q.C + 63) / 64), (unsigned)bands.n), dim3(kBlock), 0, stream, bands, B, hy);
        MYEA_HIP_TRY(hipGetLastError());
    }
    hipLaunchKernelGGL(lstm_norm_apply_kernel, dim3(grid_for(B * q.C, kBlock, 2048), (unsigned)bands.n), dim3(kBlock), 0, stream, bands, B, training ? 1 : 0, q.renorm ? 1 : 0);
    MYEA_HIP_TRY(hipGetLastError());
    prof_end((double)bands.n * (double)B * (double)q.C * sizeof(float) * 3.0);
    return MYEA_OK;
}

int Net::lstm_norm_backward_groups(LstmLayer &q, size_t B, size_t t, std::initializer_list<int> groups)
{
    NormBands bands{};
    for (int g : groups) bands.g[bands.n++] = norm_band(q, parameters, gradient, d.total_normalized_units, g, t, d.number_recurrent_depth, d.batch_size);
    if (bands.n == 0 || B == 0) return MYEA_OK;
    prof_begin(kProfNormalization);
    hipLaunchKernelGGL(lstm_norm_backward_sums_kernel, dim3((unsigned)((q.C + 63) / 64), (unsigned)bands.n), dim3(kBlock), 0, stream, bands, B, q.renorm ? 1 : 0);
    MYEA_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(lstm_norm_backward_apply_kernel, dim3(grid_for(B * q.C, kBlock, 2048), (unsigned)bands.n), dim3(kBlock), 0, stream, bands, B, q.renorm ? 1 : 0);
    MYEA_HIP_TRY(hipGetLastError());
    prof_end((double)bands.n * (double)B * (double)q.C * sizeof(float) * 5.0);
    return MYEA_OK;
}

// The s-th time step of a normalised layer: Forward_Pass__LSTM (NN/Neural_Network__Forward_Pass__OpenMP.cpp:1769-2340).
// The output gate's two sums are normalised together with the others (they depend on nothing the step computes); at the
// direction's first step only groups 0, 3, 2 and 7 run.
int Net::lstm_forward_step_norm(LstmLayer &q, size_t B, size_t s)
{
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size, C = q.C, G = q.G;
    const float *bias = parameters + q.bias;
    const size_t t = q.reverse ? T - 1 - s : s, tp = q.reverse ? t + 1 : t - 1;
    const bool first = s == 0;
    const bool zone = q.zone_state != nullptr && state == MYEA_STATE_TRAINING;
    const uint8_t *zs = zone ? q.zone_state + t * q.zone_stride : nullptr, *zo = zone ? q.zone_output + t * q.zone_stride : nullptr;
    if (!first) {   // recurrent sums h[tp] Wrec^T
        GemmParams g{};
        g.A = q.h + tp * Bmax * C; g.lda = (long)C; g.a_k_contiguous = 1;
        g.B = q.Wrec; g.ldb = (long)C; g.b_k_contiguous = 1;
        g.C = q.srec + t * Bmax * G; g.ldc = (long)G;
        g.M = (int)B; g.N = (int)G; g.K = (int)C;
        MYEA_TRY(launch_gemm(stream, g));
    }
    if (lstm_norm_fused_allowed(B, C, T)) {   // everything behind the contraction in one launch
        const NormStepArgs ns = norm_step_args(q, parameters, gradient, d.total_normalized_units, t, T, Bmax);
        const bool training = state >= MYEA_STATE_TRAINING;
        const NormHyper hy{h.normalization_epsilon, h.normalization_momentum_average, h.batch_renormalization_r_correction_maximum,
                           h.batch_renormalization_d_correction_maximum, q.renorm ? 1 : 0};
        float *acts = q.acts + t * Bmax * G, *c = q.c + t * Bmax * C, *ca = q.ca + t * Bmax * C, *hh = q.h + t * Bmax * C;
        const float *c_prev = first ? nullptr : q.c + tp * Bmax * C, *h_prev = first ? nullptr : q.h + tp * Bmax * C;
        const int tr = training ? 1 : 0;
        prof_begin(kProfNormalization);
        // few cells a workgroup when the layer is narrow (more workgroups), and no more lanes than the batch has rows for them:
        // a lane without a row still takes part in every fold
        auto launch = [&](auto kernel, int cw, int lanes) {
            hipLaunchKernelGGL(kernel, dim3((unsigned)((C + cw - 1) / cw)), dim3(lanes), 0, stream, ns, B, tr, hy, bias, (const float *)q.peep, c_prev, acts, c, ca, hh, h_prev, zs, zo);
        };
        auto pick = [&](auto first_step) {
            constexpr bool kFirst = decltype(first_step)::value;
            if (C >= 1024) {
                if (B * 16 <= 512) launch(lstm_norm_forward_fused_kernel<kFirst, 16, 512>, 16, 512); else launch(lstm_norm_forward_fused_kernel<kFirst, 16, 1024>, 16, 1024);
            } else {
                if (B * 4 <= 512) launch(lstm_norm_forward_fused_kernel<kFirst, 4, 512>, 4, 512); else launch(lstm_norm_forward_fused_kernel<kFirst, 4, 1024>, 4, 1024);
            }
        };
        if (first) pick(std::true_type{}); else pick(std::false_type{});
        MYEA_HIP_TRY(hipGetLastError());
        prof_end((double)(first ? 4 : 9) * (double)B * (double)C * sizeof(float) * 3.0);
        return MYEA_OK;
    }
    if (!first) {
        MYEA_TRY(lstm_norm_forward_groups(q, B, t, {0, 3, 5, 1, 4, 6, 7, 8}));
    } else {
        MYEA_TRY(lstm_norm_forward_groups(q, B, t, {0, 3, 7}));
    }
    const unsigned grid = grid_for(B * C, kBlock, 8192);
    hipLaunchKernelGGL(lstm_norm_gates_kernel, dim3(grid), dim3(kBlock), 0, stream, C, B, first ? 1 : 0, bias, q.peep, q.nin + t * Bmax * G, q.nrec + t * Bmax * G,
                       first ? nullptr : q.c + tp * Bmax * C, q.acts + t * Bmax * G, q.c + t * Bmax * C, zs);
    MYEA_HIP_TRY(hipGetLastError());
    MYEA_TRY(lstm_norm_forward_groups(q, B, t, {2}));
    hipLaunchKernelGGL(lstm_norm_output_kernel, dim3(grid), dim3(kBlock), 0, stream, C, B, first ? 1 : 0, bias, q.peep, q.nin + t * Bmax * G, q.nrec + t * Bmax * G,
                       q.nc + t * Bmax * C, q.c + t * Bmax * C, q.acts + t * Bmax * G, q.ca + t * Bmax * C, q.h + t * Bmax * C,
                       first ? nullptr : q.h + tp * Bmax * C, zo);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// The same time step of the backward pass (NN/Neural_Network__Recurrent_Backward_Pass__OpenMP.cpp:476-862); s counts down.
int Net::lstm_backward_step_norm(LstmLayer &q, size_t B, size_t s)
{
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size, C = q.C, G = q.G;
    const size_t t = q.reverse ? T - 1 - s : s, tn = q.reverse ? t - 1 : t + 1, tp = q.reverse ? t + 1 : t - 1;
    const bool last = s == T - 1, first = s == 0;
    int nparts = 0;
    if (!last) {   // dh[t] += (deltas of the recurrent sums of step tn) Wrec
        GemmParams g{};
        g.A = q.drec + tn * Bmax * G; g.lda = (long)G; g.a_k_contiguous = 1;
        g.B = q.Wrec; g.ldb = (long)C; g.b_k_contiguous = 0;
        g.C = q.part; g.ldc = (long)C;
        g.M = (int)B; g.N = (int)C; g.K = (int)G;
        nparts = gemm_split_k(g.M, g.N, g.K);
        if (nparts > 16) nparts = 16;   // what the slab buffer holds and the kernels below read
        g.split_k = nparts; g.split_k_slab = (long)(B * C);
        MYEA_TRY(launch_gemm(stream, g));
    }
    if (lstm_norm_fused_allowed(B, C, T)) {
        const NormStepArgs ns = norm_step_args(q, parameters, gradient, d.total_normalized_units, t, T, Bmax);
        const float *acts_next = last ? nullptr : q.acts + tn * Bmax * G, *c_prev = first ? nullptr : q.c + tp * Bmax * C;
        const float *dG_next = last ? nullptr : q.dG + tn * Bmax * G, *dc_next = last ? nullptr : q.dc + tn * Bmax * C;
        prof_begin(kProfNormalization);
        auto launch = [&](auto kernel, int cw) {
            hipLaunchKernelGGL(kernel, dim3((unsigned)((C + cw - 1) / cw)), dim3(kNormBackThreads), 0, stream, ns, B, last ? 1 : 0, q.renorm ? 1 : 0, (const float *)q.peep,
                               (const float *)(q.acts + t * Bmax * G), acts_next, (const float *)(q.ca + t * Bmax * C), c_prev, q.dh + t * Bmax * C, (const float *)q.part, nparts,
                               q.dG + t * Bmax * G, dG_next, q.dc + t * Bmax * C, dc_next, q.din + t * Bmax * G, q.drec + t * Bmax * G);
        };
        if (C >= 1024) { if (first) launch(lstm_norm_backward_fused_kernel<true, 16>, 16); else launch(lstm_norm_backward_fused_kernel<false, 16>, 16); }
        else { if (first) launch(lstm_norm_backward_fused_kernel<true, 4>, 4); else launch(lstm_norm_backward_fused_kernel<false, 4>, 4); }
        MYEA_HIP_TRY(hipGetLastError());
        prof_end((double)(first ? 4 : 9) * (double)B * (double)C * sizeof(float) * 5.0);
        return MYEA_OK;
    }
    const unsigned grid = grid_for(B * C, kBlock, 8192);
    hipLaunchKernelGGL(lstm_norm_backward_output_kernel, dim3(grid), dim3(kBlock), 0, stream, C, B, first ? 1 : 0, q.acts + t * Bmax * G, q.ca + t * Bmax * C,
                       q.dh + t * Bmax * C, q.part, nparts, q.dG + t * Bmax * G, q.din + t * Bmax * G, q.drec + t * Bmax * G, q.dc + t * Bmax * C);
    MYEA_HIP_TRY(hipGetLastError());
    if (first) MYEA_TRY(lstm_norm_backward_groups(q, B, t, {7, 2}));
    else MYEA_TRY(lstm_norm_backward_groups(q, B, t, {7, 8, 2}));
    hipLaunchKernelGGL(lstm_norm_backward_gates_kernel, dim3(grid), dim3(kBlock), 0, stream, C, B, (first && last) ? 0 : 1, first ? 1 : 0, last ? 1 : 0, q.peep,
                       q.acts + t * Bmax * G, last ? nullptr : q.acts + tn * Bmax * G, first ? nullptr : q.c + tp * Bmax * C, q.dG + t * Bmax * G,
                       last ? nullptr : q.dG + tn * Bmax * G, q.dc + t * Bmax * C, last ? nullptr : q.dc + tn * Bmax * C, q.din + t * Bmax * G, q.drec + t * Bmax * G);
    MYEA_HIP_TRY(hipGetLastError());
    if (first) MYEA_TRY(lstm_norm_backward_groups(q, B, t, {0, 3}));
    else MYEA_TRY(lstm_norm_backward_groups(q, B, t, {0, 3, 5, 1, 4, 6}));
    return MYEA_OK;
}

bool Net::lstm_backward_loop_leaves_room(size_t li, size_t B)
{
    const DevLayer &o = L[li];
    if (!o.lstm) return false;
    LstmResidentPlan plan;
    if (lstm_resident_plan(o.lstm->C, o.lstm->cpb, B, o.lstm2 ? 2 : 1, &plan) != MYEA_OK || !plan.ok || !plan.backward) return false;
    return 2 * plan.grid <= plan.cus;
}

int Net::side_stream_create()
{
    if (side_stream || side_stream_disabled()) return MYEA_OK;
    MYEA_HIP_TRY(hipStreamCreateWithFlags(&side_stream, hipStreamNonBlocking));
    MYEA_HIP_TRY(hipEventCreateWithFlags(&fork_event, hipEventDisableTiming));
    MYEA_HIP_TRY(hipEventCreateWithFlags(&join_event, hipEventDisableTiming));
    MYEA_HIP_TRY(hipEventCreateWithFlags(&update_event, hipEventDisableTiming));
    return MYEA_OK;
}

int Net::side_stream_join()
{
    if (side_stream) MYEA_HIP_TRY(hipStreamWaitEvent(stream, join_event, 0));
    return MYEA_OK;
}

// One pair of timing events brackets a whole time loop: a pair per step costs more than the 10 us steps it would time.
// Two directions: their steps are enqueued alternately, the second direction's on the side stream, so that neither
// direction's launches wait behind the other's on the host; the event pair then brackets both loops.
int Net::lstm_resident_dirs(DevLayer &o, LstmResidentDir *dirs)
{
    const bool zone = state == MYEA_STATE_TRAINING;   // zoneout acts strictly in the training state
    int n = 0;
    for (LstmLayer *q : {o.lstm, o.lstm2}) {
        if (!q) continue;
        LstmResidentDir r{};
        r.Wrec = q->Wrec; r.WrecT = q->WrecT; r.bias = parameters + q->bias; r.peep = q->peep;
        r.acts = q->acts; r.c = q->c; r.ca = q->ca; r.h = q->h;
        r.dh = q->dh; r.dG = q->dG; r.dc = q->dc; r.sums = q->sums;
        r.zone_state = zone ? q->zone_state : nullptr; r.zone_output = zone ? q->zone_output : nullptr; r.zone_stride = q->zone_stride;
        r.reverse = q->reverse ? 1 : 0;
        dirs[n++] = r;
    }
    return n;
}

int Net::lstm_forward_layer(size_t li, size_t B)
{
    DevLayer &o = L[li];
    const size_t T = d.number_recurrent_depth;
    const double loop_work = 2.0 * (double)(T - 1) * (double)B * (double)o.lstm->G * (double)o.lstm->C;   // the recurrent contractions of steps 1 .. T-1
    if (T > 1 && o.lstm->fused && !resident_off && resident_sync) {
        // the whole time loop (both directions) as one launch when the layer's shape and the device allow it
        LstmResidentPlan plan;
        const int dirs = o.lstm2 ? 2 : 1;
        MYEA_TRY(lstm_resident_plan(o.lstm->C, o.lstm->cpb, B, dirs, &plan));
        if (plan.ok) {
            MYEA_TRY(lstm_forward_inputs(li, *o.lstm, B));
            if (o.lstm2) MYEA_TRY(lstm_forward_inputs(li, *o.lstm2, B));
            LstmResidentDir rd[2];
            lstm_resident_dirs(o, rd);
            prof_begin(kProfLstmForwardLoop);
            MYEA_TRY(launch_lstm_resident_forward(stream, plan, T, B, d.batch_size, o.lstm->C, dirs, rd, resident_sync, resident_flag, fault));
            prof_end(dirs * loop_work, 1);
            if (!o.lstm2) return MYEA_OK;
            const size_t rows = (size_t)d.number_recurrent_depth * d.batch_size;
            return launch_padded_add(stream, rows, o.H, o.lstm->h, o.H, 0, o.lstm2->h, o.H, 0, o.values);  // output = h_forward + h_backward
        }
    }
    if (o.lstm->norm) {   // a normalised layer: every step is a sequence of launches; the directions run one after the other
        for (LstmLayer *q : {o.lstm, o.lstm2}) {
            if (!q) continue;
            MYEA_TRY(lstm_forward_inputs(li, *q, B));
            for (size_t s = 0; s < T; ++s) MYEA_TRY(lstm_forward_step_norm(*q, B, s));
        }
        if (!o.lstm2) return MYEA_OK;
        return launch_padded_add(stream, (size_t)d.number_recurrent_depth * d.batch_size, o.H, o.lstm->h, o.H, 0, o.lstm2->h, o.H, 0, o.values);
    }
    if (!o.lstm2) {
        MYEA_TRY(lstm_forward_inputs(li, *o.lstm, B));
        if (T > 1) prof_begin(kProfLstmForwardLoop);
        for (size_t s = 0; s < T; ++s) MYEA_TRY(lstm_forward_step(*o.lstm, B, s));
        if (T > 1) prof_end(loop_work, T - 1);
        return MYEA_OK;
    }
    {
        SideStreamScope side(*this);
        MYEA_TRY(lstm_forward_inputs(li, *o.lstm2, B));
        if (side.active) std::swap(stream, side_stream);   // back on the caller's stream while the scope stays open
        int rc = lstm_forward_inputs(li, *o.lstm, B);
        if (T > 1) prof_begin(kProfLstmForwardLoop);
        for (size_t s = 0; s < T && rc == MYEA_OK; ++s) {
            if (side.active) std::swap(stream, side_stream);
            rc = lstm_forward_step(*o.lstm2, B, s);
            if (side.active) std::swap(stream, side_stream);
            if (rc == MYEA_OK) rc = lstm_forward_step(*o.lstm, B, s);
        }
        if (side.active) std::swap(stream, side_stream);   // the scope's end expects the side stream in place
        MYEA_TRY(rc);
    }
    MYEA_TRY(side_stream_join());
    if (T > 1) prof_end(2.0 * loop_work, 2 * (T - 1));
    const size_t rows = (size_t)d.number_recurrent_depth * d.batch_size;
    return launch_padded_add(stream, rows, o.H, o.lstm->h, o.H, 0, o.lstm2->h, o.H, 0, o.values);  // output = h_forward + h_backward
}

// Recurrent__Backward_Pass__Gradient__LSTM (NN/Neural_Network__Recurrent_Backward_Pass__OpenMP.cpp:440-862), time
// descending; o.neuron_errors (= delta of the cell outputs) already holds what the layers above sent down.
// `s` counts down from T - 1: the s-th time step of the direction's own order.
int Net::lstm_backward_step(LstmLayer &q, size_t B, size_t s)
{
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size;
    // tn / tp: the steps processed after / before t in the direction's own order
    const size_t t = q.reverse ? T - 1 - s : s, tn = q.reverse ? t - 1 : t + 1, tp = q.reverse ? t + 1 : t - 1;
    float *dh_t = q.dh + t * Bmax * q.C;
    const bool last = s == T - 1, first = s == 0;
    int nparts = 0;
    if (!last && q.fused) {   // dh[t] += dG[tn] Wrec and the gate deltas of step t in one launch
        LstmFusedBackward f{};
        f.B = B; f.C = q.C; f.first_step = first;
        f.dG_next = q.dG + tn * Bmax * q.G; f.WrecT = q.WrecT; f.peep = q.peep;
        f.acts = q.acts + t * Bmax * q.G; f.acts_next = q.acts + tn * Bmax * q.G;
        f.c_prev = first ? nullptr : q.c + tp * Bmax * q.C; f.ca = q.ca + t * Bmax * q.C;
        f.dh = dh_t; f.dG = q.dG + t * Bmax * q.G; f.dc = q.dc + t * Bmax * q.C; f.dc_next = q.dc + tn * Bmax * q.C;
        return launch_lstm_fused_backward(stream, f);
    }
    if (!last) {  // Backward_Pass__LSTM_Derivative__Output, recurrent part (:1174-1226)
        GemmParams g{};
        g.A = q.dG + tn * Bmax * q.G; g.lda = (long)q.G; g.a_k_contiguous = 1;
        g.B = q.Wrec; g.ldb = (long)q.C; g.b_k_contiguous = 0;
        g.C = q.part; g.ldc = (long)q.C;
        g.M = (int)B; g.N = (int)q.C; g.K = (int)q.G;
        nparts = gemm_split_k(g.M, g.N, g.K);
        g.split_k = nparts; g.split_k_slab = (long)(B * q.C);
        MYEA_TRY(launch_gemm(stream, g));
    }
    const int mode = (first && last) ? 0 : (last ? 1 : (first ? 3 : 2));
    hipLaunchKernelGGL(lstm_backward_step_kernel, dim3(grid_for(B * q.K, kBlock, 8192)), dim3(kBlock), 0, stream, geom_of(q), B, mode, q.peep,
                       q.acts + t * Bmax * q.G, last ? nullptr : q.acts + tn * Bmax * q.G, first ? nullptr : q.c + tp * Bmax * q.C,
                       q.ca + t * Bmax * q.C, dh_t, q.dG + t * Bmax * q.G, last ? nullptr : q.dG + tn * Bmax * q.G,
                       q.dc + t * Bmax * q.C, last ? nullptr : q.dc + tn * Bmax * q.C, q.part, nparts);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int Net::lstm_backward_layer(size_t li, size_t B)
{
    DevLayer &o = L[li];
    const size_t T = d.number_recurrent_depth;
    const double loop_work = 2.0 * (double)(T - 1) * (double)B * (double)o.lstm->G * (double)o.lstm->C;
    auto seed = [&](LstmLayer &q) -> int {   // both directions start from the same delta of the layer's output
        if (q.own_h)
            MYEA_HIP_TRY(hipMemcpyAsync(q.dh, o.neuron_errors, (size_t)d.number_recurrent_depth * d.batch_size * q.C * sizeof(float), hipMemcpyDeviceToDevice, stream));
        return MYEA_OK;
    };
    for (LstmLayer *q : {o.lstm, o.lstm2})
        if (q) q->sums_groups = 0;   // the gate deltas are about to change
    if (T > 1 && o.lstm->fused && !resident_off && resident_sync) {
        LstmResidentPlan plan;
        const int dirs = o.lstm2 ? 2 : 1;
        MYEA_TRY(lstm_resident_plan(o.lstm->C, o.lstm->cpb, B, dirs, &plan));
        if (plan.ok && plan.backward) {   // the whole backward time loop (both directions) as one launch
            // weight contractions are about to run beside this loop: the form that leaves them room in LDS
            if (loop_shares_device && plan.ksplit_available) plan.ksplit = true;
            MYEA_TRY(seed(*o.lstm));
            if (o.lstm2) MYEA_TRY(seed(*o.lstm2));
            LstmResidentDir rd[2];
            lstm_resident_dirs(o, rd);
            prof_begin(kProfLstmBackwardLoop);
            MYEA_TRY(launch_lstm_resident_backward(stream, plan, T, B, d.batch_size, o.lstm->C, dirs, rd, resident_sync, resident_flag, fault, resident_exchange, resident_exchange_floats));
            prof_end(dirs * loop_work, 1);
            for (LstmLayer *q : {o.lstm, o.lstm2})
                if (q && q->sums) { q->sums_groups = (size_t)plan.row_groups; q->sums_batch = B; }
            return MYEA_OK;
        }
    }
    if (o.lstm->norm) {
        for (LstmLayer *q : {o.lstm, o.lstm2}) {
            if (!q) continue;
            MYEA_TRY(seed(*q));
            for (size_t s = T; s-- > 0;) MYEA_TRY(lstm_backward_step_norm(*q, B, s));
        }
        return MYEA_OK;
    }
    if (!o.lstm2) {
        MYEA_TRY(seed(*o.lstm));
        if (T > 1) prof_begin(kProfLstmBackwardLoop);
        for (size_t s = T; s-- > 0;) MYEA_TRY(lstm_backward_step(*o.lstm, B, s));
        if (T > 1) prof_end(loop_work, T - 1);
        return MYEA_OK;
    }
    {
        SideStreamScope side(*this);
        MYEA_TRY(seed(*o.lstm2));
        if (side.active) std::swap(stream, side_stream);
        int rc = seed(*o.lstm);
        if (T > 1) prof_begin(kProfLstmBackwardLoop);
        for (size_t s = T; s-- > 0 && rc == MYEA_OK;) {
            if (side.active) std::swap(stream, side_stream);
            rc = lstm_backward_step(*o.lstm2, B, s);
            if (side.active) std::swap(stream, side_stream);
            if (rc == MYEA_OK) rc = lstm_backward_step(*o.lstm, B, s);
        }
        if (side.active) std::swap(stream, side_stream);
        MYEA_TRY(rc);
    }
    MYEA_TRY(side_stream_join());
    if (T > 1) prof_end(2.0 * loop_work, 2 * (T - 1));
    return MYEA_OK;
}

// the operands of "delta of the layer below = dG Win" (Backward_Pass__LSTM, :1024-1120), handed to the shared driver
void Net::lstm_delta_source(size_t gi, int direction, const float **delta, size_t *width, const float **weights)
{
    LstmLayer &q = direction ? *L[gi].lstm2 : *L[gi].lstm;
    *delta = q.norm ? q.din : q.dG;   // a normalised layer hands down the deltas of its sums from below (Layer::Get__Array_Deltas__*__Input)
    *width = q.G;
    *weights = q.Win;
}

// Recurrent__Update_Derivative_Weight__LSTM (NN/Neural_Network__Recurrent_Update_Derivative_Weight__OpenMP.cpp:492-728)
// and __LSTM__Bias (:730-776).
// The weight gradients of an LSTM layer come in two independent parts that write different slots of the gradient:
// the contractions (input and recurrent weights, matrix-pipe bound) and the column reductions (peepholes and biases,
// memory bound).  `reductions` selects the part; the caller runs the reductions of all layers beside the contractions.
int Net::lstm_update_derivative_weight(size_t li, size_t B, bool reductions)
{
    for (LstmLayer *q : {L[li].lstm, L[li].lstm2}) {
        if (!q) continue;
        if (reductions) MYEA_TRY(lstm_update_derivative_weight_reductions(*q, B));
        else MYEA_TRY(lstm_update_derivative_weight_direction(li, *q, B));
    }
    return MYEA_OK;
}

int Net::lstm_update_derivative_weight_direction(size_t li, LstmLayer &q, size_t B)
{
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size;
    const float *x = layer_outputs(L[li].prev);
    const LstmGeom geom = geom_of(q);
    const bool per_t = T > 1 && B != Bmax;
    // input weights: dG^T X over every (t, b).  M x N is small and K = T*B is long: split K into slabs so that the
    // launch fills the chip; the scatter kernel sums the slabs in order.
    int s_in = 1, s_rec = 0;
    // a normalised layer: the weights from below take the deltas of the sums from below, the recurrent weights those of the
    // recurrent sums (:563-598)
    const float *d_below = q.norm ? q.din : q.dG, *d_rec = q.norm ? q.drec : q.dG;
    if (!per_t) {
        const size_t rows = T * B;
        GemmParams g{};
        g.A = d_below; g.lda = (long)q.G; g.a_k_contiguous = 0;
        g.B = x; g.ldb = (long)q.In; g.b_k_contiguous = 0;
        g.C = q.gWin; g.ldc = (long)q.In;
        g.M = (int)q.G; g.N = (int)q.In; g.K = (int)rows;
        s_in = gemm_split_k(g.M, g.N, g.K);
        g.split_k = s_in; g.split_k_slab = (long)(q.G * q.In);
        prof_begin(2);
        MYEA_TRY(launch_gemm(stream, g));
        prof_end(2.0 * (double)rows * (double)q.G * (double)q.In);
    } else {
        for (size_t c = 0; c < T; ++c) {
            GemmParams g{};
            g.A = d_below + c * Bmax * q.G; g.lda = (long)q.G; g.a_k_contiguous = 0;
            g.B = x + c * Bmax * q.In; g.ldb = (long)q.In; g.b_k_contiguous = 0;
            g.C = q.gWin; g.ldc = (long)q.In; g.accumulate = c > 0;
            g.M = (int)q.G; g.N = (int)q.In; g.K = (int)B;
            prof_begin(2);
            MYEA_TRY(launch_gemm(stream, g));
            prof_end(2.0 * (double)B * (double)q.G * (double)q.In);
        }
    }
    // recurrent weights: dG[t+1]^T h[t] for t < T-1 (second direction: dG[t]^T h[t+1]); both operand ranges are contiguous
    const size_t dg_shift = q.reverse ? 0 : 1, h_shift = q.reverse ? 1 : 0;
    if (T > 1 && !per_t) {
        const size_t rows = (T - 1) * B;
        GemmParams g{};
        g.A = d_rec + dg_shift * Bmax * q.G; g.lda = (long)q.G; g.a_k_contiguous = 0;
        g.B = q.h + h_shift * Bmax * q.C; g.ldb = (long)q.C; g.b_k_contiguous = 0;
        g.C = q.gWrec; g.ldc = (long)q.C;
        g.M = (int)q.G; g.N = (int)q.C; g.K = (int)rows;
        s_rec = gemm_split_k(g.M, g.N, g.K);
        g.split_k = s_rec; g.split_k_slab = (long)(q.G * q.C);
        if (q.pair_partials && s_rec == 1) pair_buffers(&g, q.pair_partials, reinterpret_cast<unsigned *>(q.pair_tickets));
        prof_begin(2);
        MYEA_TRY(launch_gemm(stream, g));
        prof_end(2.0 * (double)rows * (double)q.G * (double)q.C);
    } else if (T > 1) {
        s_rec = 1;
        for (size_t c = 0; c + 1 < T; ++c) {
            GemmParams g{};
            g.A = d_rec + (c + dg_shift) * Bmax * q.G; g.lda = (long)q.G; g.a_k_contiguous = 0;
            g.B = q.h + (c + h_shift) * Bmax * q.C; g.ldb = (long)q.C; g.b_k_contiguous = 0;
            g.C = q.gWrec; g.ldc = (long)q.C; g.accumulate = c > 0;
            g.M = (int)q.G; g.N = (int)q.C; g.K = (int)B;
            prof_begin(2);
            MYEA_TRY(launch_gemm(stream, g));
            prof_end(2.0 * (double)B * (double)q.G * (double)q.C);
        }
    }
    hipLaunchKernelGGL(lstm_scatter_add_kernel, dim3((unsigned)q.G), dim3(kBlock), 0, stream, geom, gradient, q.gWin, s_in, q.gWrec, s_rec);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

// MYEA_LSTM_RESIDENT_SUMS=0: the bias and peephole gradients always come from their own pass over the gate deltas
static bool resident_sums_allowed()
{
    const char *e = std::getenv("MYEA_LSTM_RESIDENT_SUMS");   // read at every call: a test compares the two ways in one process
    return !(e && e[0] == '0');
}

int Net::lstm_update_derivative_weight_reductions(LstmLayer &q, size_t B)
{
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size;
    const LstmGeom geom = geom_of(q);
    if (T * B > 0xffffffffull) { set_last_error("LSTM weight gradients: %zu x %zu (time steps x batch) rows do not fit 32 bits", T, B); return MYEA_E_INVALID; }
    if (q.sums_groups && q.sums_batch == B && resident_sums_allowed()) {   // the backward time loop summed them as it went
        hipLaunchKernelGGL(lstm_bias_peep_final_kernel, dim3(grid_for(7 * q.C, kBlock)), dim3(kBlock), 0, stream, geom, q.sums_groups, q.sums, gradient + q.bias, gradient);
        MYEA_HIP_TRY(hipGetLastError());
        return MYEA_OK;
    }
    if (q.cpb == 1) {   // biases and peepholes in one pass over the gate deltas
        const size_t colblocks = (q.C + 63) / 64;
        size_t S = (512 + colblocks - 1) / colblocks;          // aim at >= 512 workgroups
        if (S > (B + 3) / 4) S = (B + 3) / 4;
        if (S > 64) S = 64;                                     // the scratch holds 64 x 7 x C partial sums
        const size_t per_lane = (B + 4 * S - 1) / (4 * S);
        S = (B + 4 * per_lane - 1) / (4 * per_lane);
        hipLaunchKernelGGL(lstm_bias_peep_partial_kernel, dim3((unsigned)colblocks, (unsigned)S), dim3(kBlock), 0, stream, q.C, B, Bmax, T, per_lane, q.reverse ? 1 : 0,
                           q.c, q.dG, q.norm ? q.drec : q.dG, q.norm ? q.din : q.dG, scratch);
        MYEA_HIP_TRY(hipGetLastError());
        hipLaunchKernelGGL(lstm_bias_peep_final_kernel, dim3(grid_for(7 * q.C, kBlock)), dim3(kBlock), 0, stream, geom, S, scratch, gradient + q.bias, gradient);
        MYEA_HIP_TRY(hipGetLastError());
        return MYEA_OK;
    }
    // peepholes
    {
        size_t S, chunk;
        split_rows(T * B, q.C, S, chunk);
        PeepF f{geom, B, Bmax, T, q.c, q.dG, q.reverse ? 1 : 0};
        hipLaunchKernelGGL((column_partial_kernel<3, PeepF>), dim3((unsigned)((q.C + 63) / 64), (unsigned)S), dim3(kBlock), 0, stream, T * B, q.C, chunk, scratch, f);
        MYEA_HIP_TRY(hipGetLastError());
        hipLaunchKernelGGL(lstm_peep_final_kernel, dim3(grid_for(3 * q.C, kBlock)), dim3(kBlock), 0, stream, geom, S, scratch, gradient);
        MYEA_HIP_TRY(hipGetLastError());
    }
    // the four bias vectors: one contiguous [G] slice in the order z | i | f | o
    {
        size_t S, chunk;
        split_rows(T * B, q.G, S, chunk);
        StridedSumF f{B, Bmax, q.G, q.dG};
        hipLaunchKernelGGL((column_partial_kernel<1, StridedSumF>), dim3((unsigned)((q.G + 63) / 64), (unsigned)S), dim3(kBlock), 0, stream, T * B, q.G, chunk, scratch, f);
        MYEA_HIP_TRY(hipGetLastError());
        hipLaunchKernelGGL(lstm_colsum_final_kernel, dim3(grid_for(q.G, kBlock)), dim3(kBlock), 0, stream, q.G, S, scratch, gradient + q.bias);
        MYEA_HIP_TRY(hipGetLastError());
    }
    return MYEA_OK;
}

const float *Net::lstm_tensor(size_t li, int kind, size_t *count)
{
    if (count) *count = 0;
    const bool backward = (kind & MYEA_TENSOR_DIRECTION_BACKWARD) != 0;
    kind &= ~MYEA_TENSOR_DIRECTION_BACKWARD;
    LstmLayer *q = backward ? L[li].lstm2 : L[li].lstm;
    if (!q) return nullptr;
    // The device keeps gate tensors packed as rows of [G]; taps are served from small staging copies.
    const size_t T = d.number_recurrent_depth, Bmax = d.batch_size, rows = T * Bmax;
    const float *src = nullptr;
    size_t width = 0, offset = 0, ld = 0;
    const int group = (kind >> MYEA_TENSOR_LSTM_NORM_GROUP_SHIFT) & 15;   // 1 + the group of normalised units, or 0
    kind &= ~(15 << MYEA_TENSOR_LSTM_NORM_GROUP_SHIFT);
    if (group) {
        if (!q->norm || group > 9) return nullptr;
        const int g = group - 1;
        const NormBand b = norm_band(*q, parameters, gradient, d.total_normalized_units, g, 0, T, Bmax);
        const size_t TH = T * q->C;
        switch (kind) {
        case MYEA_TENSOR_NORM_MEANS: if (count) *count = TH; return b.mean;
        case MYEA_TENSOR_NORM_VARIANCES: if (count) *count = TH; return b.sigma;
        case MYEA_TENSOR_NORM_MEANS_AVERAGES: if (count) *count = TH; return b.mean_avg;
        case MYEA_TENSOR_NORM_VARIANCES_AVERAGES: if (count) *count = TH; return b.sigma_avg;
        case MYEA_TENSOR_NORM_HATS: src = b.hat; ld = b.ldo; break;
        case MYEA_TENSOR_ERRORS: src = b.d; ld = b.ldd; break;
        default: return nullptr;
        }
        if (hipMemcpy2DAsync(tmp1, q->C * sizeof(float), src, ld * sizeof(float), q->C * sizeof(float), rows, hipMemcpyDeviceToDevice, stream) != hipSuccess) return nullptr;
        if (count) *count = rows * q->C;
        return tmp1;
    }
    switch (kind) {
    case MYEA_TENSOR_LSTM_CELL_OUTPUT: if (count) *count = rows * q->C; return q->h;
    case MYEA_TENSOR_LSTM_DELTA_CELL_OUTPUT: if (count) *count = rows * q->C; return q->dh;
    case MYEA_TENSOR_LSTM_CELL_STATE: if (count) *count = rows * q->C; return q->c;
    case MYEA_TENSOR_LSTM_DELTA_CELL_STATE: if (count) *count = rows * q->C; return q->dc;
    case MYEA_TENSOR_LSTM_CELL_INPUT: src = q->acts; width = q->C; offset = 0; break;
    case MYEA_TENSOR_LSTM_INPUT_GATE: src = q->acts; width = q->K; offset = q->C; break;
    case MYEA_TENSOR_LSTM_FORGET_GATE: src = q->acts; width = q->K; offset = q->C + q->K; break;
    case MYEA_TENSOR_LSTM_OUTPUT_GATE: src = q->acts; width = q->K; offset = q->C + 2 * q->K; break;
    case MYEA_TENSOR_LSTM_DELTA_CELL_INPUT: src = q->dG; width = q->C; offset = 0; break;
    case MYEA_TENSOR_LSTM_DELTA_INPUT_GATE: src = q->dG; width = q->K; offset = q->C; break;
    case MYEA_TENSOR_LSTM_DELTA_FORGET_GATE: src = q->dG; width = q->K; offset = q->C + q->K; break;
    case MYEA_TENSOR_LSTM_DELTA_OUTPUT_GATE: src = q->dG; width = q->K; offset = q->C + 2 * q->K; break;
    default: return nullptr;
    }
    ld = q->G;
    // strided copy of the column band into tmp1 (large enough: rows * max width)
    if (hipMemcpy2DAsync(tmp1, width * sizeof(float), src + offset, ld * sizeof(float), width * sizeof(float), rows, hipMemcpyDeviceToDevice, stream) != hipSuccess) return nullptr;
    if (count) *count = rows * width;
    return tmp1;
}

// the running mean / sigma of one group of a normalised layer, writable (a checkpoint restores them)
float *Net::lstm_norm_statistics(size_t li, int kind, size_t *count)
{
    if (count) *count = 0;
    const bool backward = (kind & MYEA_TENSOR_DIRECTION_BACKWARD) != 0;
    kind &= ~MYEA_TENSOR_DIRECTION_BACKWARD;
    LstmLayer *q = backward ? L[li].lstm2 : L[li].lstm;
    const int group = (kind >> MYEA_TENSOR_LSTM_NORM_GROUP_SHIFT) & 15;
    kind &= ~(15 << MYEA_TENSOR_LSTM_NORM_GROUP_SHIFT);
    if (!q || !q->norm || group < 1 || group > 9) return nullptr;
    const size_t TH = d.number_recurrent_depth * q->C;
    if (count) *count = TH;
    if (kind == MYEA_TENSOR_NORM_MEANS_AVERAGES) return q->stats[group - 1] + 2 * TH;
    if (kind == MYEA_TENSOR_NORM_VARIANCES_AVERAGES) return q->stats[group - 1] + 3 * TH;
    return nullptr;
}

}  // namespace myea
