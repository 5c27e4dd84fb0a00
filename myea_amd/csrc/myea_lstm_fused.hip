// myea_lstm_fused.hip — one launch per LSTM time step: the recurrent contraction and all gate math of the step.
//
// The per-step recurrent products are skinny (batch x 4C x C forward, batch x C x 4C backward: 0.5 GFLOP at C = 512,
// batch 256) and sit on the critical path of the time loop, T times per layer and pass.  As a generic contraction
// plus a gate kernel they cost two launches and a round trip of split-K slabs through memory per step.  Here one
// workgroup owns a small output tile whose columns are ALL FOUR gates of the same 16 cells, its four wavefronts split
// the k range between them, the partial tiles meet in LDS, and the same workgroup finishes the step: activations,
// cell state, output (forward) or the gate deltas (backward).  Tiles are sized so that a step launches >= 256
// workgroups at batch 256.  No operand is shared between wavefronts, so each wavefront stages its own [rows][32 k]
// tiles: global -> LDS directly (global_load_lds_dwordx4, 8 lanes per 128-byte row segment - a lane-per-row register
// load would spend a tag lookup per lane), 16-byte chunks XOR-swizzled by (row >> 1) & 7 so that the ds_read_b128
// fragment reads spread over the banks; a wavefront only reads what it loaded itself, so the pipeline needs no
// barrier, only vmcnt.
//
// Layout requirements (checked on the host): one cell per block (K == C, G == 4C) and C a multiple of 32.
// Everything else runs on the generic path (contraction + lstm_*_step_kernel).
//
// MFMA operand layouts used below (k may be permuted freely as long as A and B agree):
//   v_mfma_f32_32x32x2_f32: lane l supplies A[row l%32][k l/32] and B[k l/32][col l%32]; accumulator register r of
//                           lane l is C[(r/4)*8 + (l/32)*4 + r%4][l%32].
//   v_mfma_f32_16x16x4_f32: lane l supplies A[row l%16][k l/16] and B[k l/16][col l%16]; accumulator register r of
//                           lane l is C[(l/16)*4 + r][l%16].
// A lane reads 16 bytes (4 consecutive k) per operand from the staged tile and feeds element j to the j-th MFMA of a
// group of four: lane group h = l/32 takes the chunk 2 g + h of the 32 k (32x32x2, g = 0..3), lane group q = l/16 the
// chunk 4 g + q (16x16x4, g = 0..1).
// Workgroup -> tile: consecutive workgroup ids land on different XCDs (8, each with its own L2); an XCD always gets the
// same cell tiles, so its slice of the recurrent weights stays in its L2 from one time step to the next.
//
// NN/ = Neural_Network_Library_Windows/Source_Files/Neural_Network/.
#include "myea_kernels.h"

namespace myea {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kFwdStages = 2, kBwdStages = 4;   // LDS stages (of 32 k) per wavefront

// One wavefront's tile of ROWS rows x 32 k in LDS, filled by ROWS / 8 direct loads of 1 KiB: lane l of load q brings
// the 16-byte chunk (l & 7) ^ swizzle of row 8 q + l / 8, and lands at byte 16 l of the load's KiB.
template <int ROWS>
struct WaveTile {
    const float *ptr[ROWS / 8];
    // row_of(r) = global row of tile row r (already clamped to the operand's extent)
    template <class RowOf>
    __device__ __forceinline__ void init(const float *base, size_t ld, size_t k0, RowOf row_of)
    {
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int q = 0; q < ROWS / 8; ++q) {
            const int r = q * 8 + (lane >> 3);
            const int chunk = (lane & 7) ^ ((r >> 1) & 7);
            ptr[q] = base + row_of(r) * ld + k0 + chunk * 4;
        }
    }
    __device__ __forceinline__ void fill(float *tile, size_t advance)
    {
#pragma unroll
        for (int q = 0; q < ROWS / 8; ++q) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)ptr[q],
                                             (__attribute__((address_space(3))) void *)(tile + q * 256), 16, 0, 0);
            ptr[q] += advance;
        }
    }
    static __device__ __forceinline__ f32x4 chunk(const float *tile, int row, int c)
    {
        return *reinterpret_cast<const f32x4 *>(tile + row * 32 + ((c ^ ((row >> 1) & 7)) << 2));
    }
};
template <int N>
__device__ __forceinline__ void wait_loads() { __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14)); }   // vmcnt(N)

// XCD x = id % 8 owns the cell tiles [x nt/8, (x+1) nt/8) when they divide evenly
__device__ __forceinline__ void tile_of(unsigned id, int ntc, int &tile_c, int &tile_r)
{
    if ((ntc & 7) == 0) {
        const int per = ntc >> 3, xcd = (int)(id & 7), idx = (int)(id >> 3);
        tile_c = xcd * per + idx % per;
        tile_r = idx / per;
    } else {
        tile_c = (int)(id % (unsigned)ntc);
        tile_r = (int)(id / (unsigned)ntc);
    }
}

__device__ __forceinline__ float sigmoid_f(float s) { return 1.f / (1.f + expf(-s)); }
__device__ __forceinline__ float tanh_f(float s) { return 2.f / (1.f + expf(-2.f * s)) - 1.f; }  // AF_TANH_real
__device__ __forceinline__ f32x4 ld4(const float *p) { return *reinterpret_cast<const f32x4 *>(p); }

// ---- forward -------------------------------------------------------------------------------------------------
// Tile: 32 examples x CELLS cells (4 CELLS gate columns z | i | f | o), CELLS = 16, or 8 where 16 would leave half of the
// compute units without a workgroup (small batches).  Wavefront w sums the k groups w, w + 4, w + 8, ...
// Gate math: Forward_Pass__LSTM__Gates_CIF_AF_State (NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:1042-1191),
// __States_AF (:1547-1582), __Output (:1351-1418), for a step that has a previous step.
template <int CELLS>
__global__ __launch_bounds__(kThreads) void lstm_fused_forward_kernel(LstmFusedForward p)
{
    constexpr int NB = 4 * CELLS;               // rows of the weight tile = gate columns of the output tile
    constexpr int PAIRS = 32 * CELLS / kThreads;   // (example, cell) pairs per lane
    constexpr int kFwdStride = NB + 8;          // floats per row of a wavefront's partial tile in LDS
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, lane32 = lane & 31, half = lane >> 5;
    const int C = (int)p.C, B = (int)p.B;
    int tile_c, tile_r;
    tile_of(blockIdx.x, C / CELLS, tile_c, tile_r);
    const int c0 = tile_c * CELLS, r0 = tile_r * 32;
    const int ng = (C / 32 - wave + 3) / 4;          // this wavefront's groups of 32 k: wave, wave + 4, wave + 8, ...
    constexpr int kStage = (32 + NB) * 32;           // floats: A tile 32 x 32, then B tile NB x 32
    float *stage0 = smem + wave * kFwdStages * kStage;

    // what the gate math of this lane's (example, cell) pairs reads does not depend on the contraction: fetch it now
    float e_in[PAIRS][4], e_bias[PAIRS][4], e_peep[PAIRS][3], e_cp[PAIRS];
#pragma unroll
    for (int q = 0; q < PAIRS; ++q) {
        const int pair = threadIdx.x + q * kThreads, row = pair / CELLS, cell = pair % CELLS;
        const int b = min(r0 + row, B - 1), k = c0 + cell;
        const float *arow = p.acts + (size_t)b * 4 * C;
#pragma unroll
        for (int gate = 0; gate < 4; ++gate) { e_in[q][gate] = arow[gate * C + k]; e_bias[q][gate] = p.bias[gate * C + k]; }
#pragma unroll
        for (int gate = 0; gate < 3; ++gate) e_peep[q][gate] = p.peep[gate * C + k];
        e_cp[q] = p.c_prev[(size_t)b * C + k];
    }

    f32x16 acc0, acc1;
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc0[r] = 0.f; acc1[r] = 0.f; }
    if (ng > 0) {
        WaveTile<32> ta;
        WaveTile<NB> tb;
        ta.init(p.h_prev, (size_t)C, (size_t)wave * 32, [&](int r) { return (size_t)min(r0 + r, B - 1); });
        // tile row j of B is gate j / CELLS of cell c0 + j % CELLS: row gate * C + cell of the packed matrix
        tb.init(p.Wrec, (size_t)C, (size_t)wave * 32, [&](int r) { return (size_t)(r / CELLS) * C + c0 + (r % CELLS); });
        ta.fill(stage0, 128);
        tb.fill(stage0 + 32 * 32, 128);
        for (int g = 0; g < ng; ++g) {
            const float *cur = stage0 + (g & 1) * kStage;
            if (g + 1 < ng) {   // the other stage was last read by the MFMAs of group g - 1
                float *nxt = stage0 + ((g + 1) & 1) * kStage;
                ta.fill(nxt, 128);
                tb.fill(nxt + 32 * 32, 128);
                wait_loads<4 + NB / 8>();   // the loads just issued may stay in flight
            } else {
                wait_loads<0>();
            }
            const float *la = cur, *lb = cur + 32 * 32;
            // fragments of k group kg + 1 are read while the MFMAs of group kg issue
            f32x4 fa[2], fb0[2], fb1[2];
            fa[0] = WaveTile<32>::chunk(la, lane32, half);
            fb0[0] = WaveTile<NB>::chunk(lb, lane32, half);
            if constexpr (NB == 64) fb1[0] = WaveTile<NB>::chunk(lb, 32 + lane32, half);
#pragma unroll
            for (int kg = 0; kg < 4; ++kg) {
                const int cb = kg & 1, nb = cb ^ 1;
                if (kg + 1 < 4) {
                    fa[nb] = WaveTile<32>::chunk(la, lane32, (kg + 1) * 2 + half);
                    fb0[nb] = WaveTile<NB>::chunk(lb, lane32, (kg + 1) * 2 + half);
                    if constexpr (NB == 64) fb1[nb] = WaveTile<NB>::chunk(lb, 32 + lane32, (kg + 1) * 2 + half);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cb][s], fb0[cb][s], acc0, 0, 0, 0);
                    if constexpr (NB == 64) acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cb][s], fb1[cb][s], acc1, 0, 0, 0);
                }
            }
        }
    }
    __syncthreads();   // every wavefront is done with its stages: the partial tiles reuse the memory
    float *part = smem;
    float *mine = part + wave * 32 * kFwdStride;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int row = (r >> 2) * 8 + half * 4 + (r & 3);
        mine[row * kFwdStride + lane32] = acc0[r];
        if constexpr (NB == 64) mine[row * kFwdStride + 32 + lane32] = acc1[r];
    }
    __syncthreads();
    // 32 x CELLS (example, cell) pairs
#pragma unroll
    for (int q = 0; q < PAIRS; ++q) {
        const int pair = threadIdx.x + q * kThreads, row = pair / CELLS, cell = pair % CELLS;
        const int b = r0 + row;
        if (b >= B) continue;
        float rec[4];
#pragma unroll
        for (int gate = 0; gate < 4; ++gate) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < 4; ++w) v += part[(w * 32 + row) * kFwdStride + gate * CELLS + cell];
            rec[gate] = v;
        }
        const int k = c0 + cell;
        float *arow = p.acts + (size_t)b * 4 * C;
        const size_t ci = (size_t)b * C + k;
        const float cp = e_cp[q];
        float si = e_in[q][1] + rec[1] + e_bias[q][1];
        float sf = e_in[q][2] + rec[2] + e_bias[q][2];
        si += cp * e_peep[q][0];
        sf += cp * e_peep[q][1];
        const float gi = sigmoid_f(si), gf = sigmoid_f(sf);
        const float z = tanh_f(e_in[q][0] + rec[0] + e_bias[q][0]);
        float cs = z * gi + gf * cp;
        if (p.zone_state && !p.zone_state[k]) cs = cp;   // zoned-out cell state: keep the previous one
        const float a = tanh_f(cs);
        const float so = e_in[q][3] + rec[3] + e_bias[q][3] + cs * e_peep[q][2];
        const float go = sigmoid_f(so);
        arow[k] = z; arow[C + k] = gi; arow[2 * C + k] = gf; arow[3 * C + k] = go;
        float hv = a * go;
        if (p.zone_output && !p.zone_output[k]) hv = p.h_prev[ci];   // zoned-out cell output
        p.c[ci] = cs; p.ca[ci] = a; p.h[ci] = hv;
    }
}

// ---- backward ------------------------------------------------------------------------------------------------
// dh[t] += dG[t'] Wrec (t' = the step processed after t), then the gate deltas of step t.
// Tile: ROWS examples x 16 cells (ROWS = 32, or 16 for small batches, as in the forward step); wavefront w sums the k
// range of gate w (k = gate * C + cell of dG[t']), reading the transposed packed matrix WrecT [C][4C] so that both
// operands are k-contiguous.
// Gate math: Backward_Pass__LSTM_Derivative__Output (NN/Neural_Network__Recurrent_Backward_Pass__OpenMP.cpp:1228-1240),
// __Cell_State_AF (:1275-1327), __Gates_CIF_AF_State (:1329-1604) for a step that has a following step; `first_step`:
// the sequence's first step writes no forget-gate delta (:1460-1534).
constexpr int kBwdStride = 17;

template <int ROWS>
__global__ __launch_bounds__(kThreads) void lstm_fused_backward_kernel(LstmFusedBackward p)
{
    constexpr int PAIRS = ROWS * 16 / kThreads;   // (example, cell) pairs per lane
    constexpr int kLoads = ROWS / 8 + 2;          // direct loads per stage and wavefront
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, lane16 = lane & 15, quad = lane >> 4;
    const int C = (int)p.C, B = (int)p.B, G = 4 * C;
    int tile_c, tile_r;
    tile_of(blockIdx.x, C / 16, tile_c, tile_r);
    const int c0 = tile_c * 16, r0 = tile_r * ROWS;
    const int ng = C / 32;   // groups of 32 k in this wavefront's range of C
    constexpr int kStage = (ROWS + 16) * 32;   // floats: A tile ROWS x 32 (rows of dG[t']), then B tile 16 x 32 (rows of WrecT)
    float *stage0 = smem + wave * kBwdStages * kStage;

    // operands of the gate math of this lane's (example, cell) pairs, fetched ahead of the contraction
    float e_dh[PAIRS], e_act[PAIRS][4], e_ca[PAIRS], e_din[PAIRS], e_dfn[PAIRS], e_fn[PAIRS], e_peep[PAIRS][3], e_dcn[PAIRS], e_cp[PAIRS];
#pragma unroll
    for (int q = 0; q < PAIRS; ++q) {
        const int pair = threadIdx.x + q * kThreads, row = pair >> 4, cell = pair & 15;
        const int b = min(r0 + row, B - 1), k = c0 + cell;
        const size_t ci = (size_t)b * C + k, gi_ = (size_t)b * G;
        e_dh[q] = p.dh[ci];
#pragma unroll
        for (int gate = 0; gate < 4; ++gate) e_act[q][gate] = p.acts[gi_ + gate * C + k];
        e_ca[q] = p.ca[ci];
        e_din[q] = p.dG_next[gi_ + C + k]; e_dfn[q] = p.dG_next[gi_ + 2 * C + k]; e_fn[q] = p.acts_next[gi_ + 2 * C + k];
#pragma unroll
        for (int gate = 0; gate < 3; ++gate) e_peep[q][gate] = p.peep[gate * C + k];
        e_dcn[q] = p.dc_next[ci];
        e_cp[q] = p.first_step ? 0.f : p.c_prev[ci];
    }

    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
    WaveTile<ROWS> ta;
    WaveTile<16> tb;
    ta.init(p.dG_next, (size_t)G, (size_t)wave * C, [&](int r) { return (size_t)min(r0 + r, B - 1); });
    tb.init(p.WrecT, (size_t)G, (size_t)wave * C, [&](int r) { return (size_t)(c0 + r); });
    // stages g + 1 .. g + 3 are in flight while group g computes
#pragma unroll
    for (int u = 0; u < kBwdStages - 1; ++u)
        if (u < ng) { ta.fill(stage0 + u * kStage, 32); tb.fill(stage0 + u * kStage + ROWS * 32, 32); }
    for (int g = 0; g < ng; ++g) {
        const float *cur = stage0 + (g & (kBwdStages - 1)) * kStage;
        if (g + kBwdStages - 1 < ng) {   // that stage was last read by the MFMAs of group g - 1
            float *nxt = stage0 + ((g + kBwdStages - 1) & (kBwdStages - 1)) * kStage;
            ta.fill(nxt, 32);
            tb.fill(nxt + ROWS * 32, 32);
            wait_loads<3 * kLoads>();
        } else if (g + 2 < ng) {
            wait_loads<2 * kLoads>();
        } else if (g + 1 < ng) {
            wait_loads<kLoads>();
        } else {
            wait_loads<0>();
        }
        const float *la = cur, *lb = cur + ROWS * 32;
        f32x4 fa0[2], fa1[2], fb[2];
#pragma unroll
        for (int kg = 0; kg < 2; ++kg) {
            fa0[kg] = WaveTile<ROWS>::chunk(la, lane16, kg * 4 + quad);
            if constexpr (ROWS == 32) fa1[kg] = WaveTile<ROWS>::chunk(la, 16 + lane16, kg * 4 + quad);
            fb[kg] = WaveTile<16>::chunk(lb, lane16, kg * 4 + quad);
        }
#pragma unroll
        for (int kg = 0; kg < 2; ++kg)
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(fa0[kg][s], fb[kg][s], acc0, 0, 0, 0);
                if constexpr (ROWS == 32) acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(fa1[kg][s], fb[kg][s], acc1, 0, 0, 0);
            }
    }
    __syncthreads();   // every wavefront is done with its stages: the partial tiles reuse the memory
    float *part = smem;
    float *mine = part + wave * ROWS * kBwdStride;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        mine[(quad * 4 + r) * kBwdStride + lane16] = acc0[r];
        if constexpr (ROWS == 32) mine[(16 + quad * 4 + r) * kBwdStride + lane16] = acc1[r];
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < PAIRS; ++q) {
        const int pair = threadIdx.x + q * kThreads, row = pair >> 4, cell = pair & 15;
        const int b = r0 + row;
        if (b >= B) continue;
        float rec = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) rec += part[(w * ROWS + row) * kBwdStride + cell];
        const int k = c0 + cell;
        const size_t ci = (size_t)b * C + k, gi_ = (size_t)b * G;
        const float dh = e_dh[q] + rec;
        p.dh[ci] = dh;
        float *drow = p.dG + gi_;
        const float z = e_act[q][0], gi = e_act[q][1], gf = e_act[q][2], go = e_act[q][3];
        const float a = e_ca[q];
        const float ddo = go * (1.f - go) * (dh * a);
        drow[3 * C + k] = ddo;
        float e = dh * go * (1.f - a * a);
        e += e_peep[q][2] * ddo;
        e += e_peep[q][0] * e_din[q];
        e += e_peep[q][1] * e_dfn[q];
        e += e_dcn[q] * e_fn[q];
        p.dc[ci] = e;
        drow[k] = e * gi * (1.f - z * z);
        drow[C + k] = (e * z) * (gi * (1.f - gi));
        drow[2 * C + k] = p.first_step ? 0.f : (e * e_cp[q]) * (gf * (1.f - gf));
    }
}

// WrecT [C][4C] <- Wrec [4C][C]
__global__ __launch_bounds__(kThreads) void transpose_kernel(size_t rows, size_t cols, const float *__restrict__ src, float *__restrict__ dst)
{
    __shared__ float tile[32][33];
    const size_t bx = (size_t)blockIdx.x * 32, by = (size_t)blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
    for (int j = ty; j < 32; j += 8)
        if (by + j < rows && bx + tx < cols) tile[j][tx] = src[(by + j) * cols + bx + tx];
    __syncthreads();
    for (int j = ty; j < 32; j += 8)
        if (bx + j < cols && by + tx < rows) dst[(bx + j) * rows + by + tx] = tile[tx][j];
}

bool aligned16(const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; }

}  // namespace

bool lstm_fused_supported(size_t C, size_t cells_per_block) { return cells_per_block == 1 && C >= 32 && C % 32 == 0 && C <= (1u << 20); }

// Half-size tiles where the full-size tiling would give at most half of the 256 compute units a workgroup (small batches):
// twice the workgroups, each with half the contraction work, and two of them fit a compute unit's LDS.
static bool narrow_tiles(size_t B, size_t C) { return ((B + 31) / 32) * (C / 16) <= 128; }

template <int CELLS>
static int launch_forward(hipStream_t s, const LstmFusedForward &p)
{
    const size_t blocks = ((p.B + 31) / 32) * (p.C / CELLS);
    if (blocks > 0x7fffffffu) { set_last_error("fused LSTM forward step: grid out of range"); return MYEA_E_INVALID; }
    constexpr size_t lds = (size_t)4 * kFwdStages * (32 + 4 * CELLS) * 32 * sizeof(float);
    static_assert(lds >= 4 * 32 * (4 * CELLS + 8) * sizeof(float), "the partial tiles reuse the stages");
    static bool attr_done = false;
    if (!attr_done) {
        MYEA_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(lstm_fused_forward_kernel<CELLS>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_done = true;
    }
    hipLaunchKernelGGL(lstm_fused_forward_kernel<CELLS>, dim3((unsigned)blocks), dim3(kThreads), lds, s, p);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_lstm_fused_forward(hipStream_t s, const LstmFusedForward &p)
{
    if (p.B == 0) return MYEA_OK;
    if (!lstm_fused_supported(p.C, 1) || !p.h_prev || !p.Wrec || !p.bias || !p.peep || !p.acts || !p.c_prev || !p.c || !p.ca || !p.h ||
        !aligned16(p.h_prev) || !aligned16(p.Wrec)) {
        set_last_error("fused LSTM forward step: unsupported shape or operand (C = %zu)", p.C);
        return MYEA_E_INVALID;
    }
    return narrow_tiles(p.B, p.C) ? launch_forward<8>(s, p) : launch_forward<16>(s, p);
}

template <int ROWS>
static int launch_backward(hipStream_t s, const LstmFusedBackward &p)
{
    const size_t blocks = ((p.B + ROWS - 1) / ROWS) * (p.C / 16);
    if (blocks > 0x7fffffffu) { set_last_error("fused LSTM backward step: grid out of range"); return MYEA_E_INVALID; }
    constexpr size_t lds = (size_t)4 * kBwdStages * (ROWS + 16) * 32 * sizeof(float);
    static_assert(lds >= 4 * ROWS * kBwdStride * sizeof(float), "the partial tiles reuse the stages");
    static bool attr_done = false;
    if (!attr_done) {
        MYEA_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(lstm_fused_backward_kernel<ROWS>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_done = true;
    }
    hipLaunchKernelGGL(lstm_fused_backward_kernel<ROWS>, dim3((unsigned)blocks), dim3(kThreads), lds, s, p);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_lstm_fused_backward(hipStream_t s, const LstmFusedBackward &p)
{
    if (p.B == 0) return MYEA_OK;
    if (!lstm_fused_supported(p.C, 1) || !p.dG_next || !p.WrecT || !p.peep || !p.acts || !p.acts_next || !p.ca || !p.dh || !p.dG || !p.dc ||
        !p.dc_next || (!p.first_step && !p.c_prev) || !aligned16(p.dG_next) || !aligned16(p.WrecT)) {
        set_last_error("fused LSTM backward step: unsupported shape or operand (C = %zu)", p.C);
        return MYEA_E_INVALID;
    }
    return narrow_tiles(p.B, p.C) ? launch_backward<16>(s, p) : launch_backward<32>(s, p);
}

int launch_transpose(hipStream_t s, size_t rows, size_t cols, const float *src, float *dst)
{
    if (rows == 0 || cols == 0) return MYEA_OK;
    hipLaunchKernelGGL(transpose_kernel, dim3((unsigned)((cols + 31) / 32), (unsigned)((rows + 31) / 32)), dim3(kThreads), 0, s, rows, cols, src, dst);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

}  // namespace myea
