// myea_gemm.hip — FP32 MFMA dense contraction for gfx950 (CDNA4), LDS-staged.
//
// One kernel template covers the three contractions of the fully-connected and LSTM path:
//   forward  Y  = X W^T          (A k-contiguous, B k-contiguous)   Forward_Pass__FC,
//            Neural_Network__Forward_Pass__OpenMP.cpp:4517-4557
//   backward dX = delta W        (A k-contiguous, B n-contiguous)   Backward_Pass__FC, Neural_Network__Backward_Pass__OpenMP.cpp:1044-1082
//   weights  dW += delta^T X     (A m-contiguous, B n-contiguous)   Update_Derivative_Weight__FC,
//            Neural_Network__Update_Derivative_Weight__OpenMP.cpp:178-216
//
// Tiling: a workgroup of 256 lanes (4 wavefronts, 2 x 2) owns a BM x BN tile of C; each wavefront owns
// (BM/2) x (BN/2) as TM x TN accumulators of v_mfma_f32_32x32x2_f32 (16 VGPRs each).  The K loop moves
// BK = 32 columns per step through LDS stages with one barrier per step; the fragments of the next 8 k's are read from
// LDS while the MFMAs of the current 8 issue.  General path (any alignment): global -> registers (guarded scalar loads,
// issued before the MFMA block of the current step) -> LDS, two stages.  Operands keep their global orientation in LDS,
// so no transposes are needed:
//   k-contiguous operand : LDS [rows][BK + 4]   fragment = one ds_read_b128 per 4 MFMA k-steps
//   mn-contiguous operand: LDS [BK][rows + 8]   fragment = conflict-free ds_read_b32 per k
// When the operands are 16-byte aligned the tiles do not pass through registers at all: global_load_lds_dwordx4 writes
// 1 KiB per wavefront instruction straight into LDS (lane l lands at base + 16 l), which rules out per-row padding, so
//   k-contiguous operand : LDS [rows][BK], the 16-byte chunk c of row r stored at chunk c ^ ((r >> 1) & 7)
//   mn-contiguous operand: LDS [BK][rows] in 1 KiB pieces, each padded so that k and k + 4 sit 32 banks apart
// both again conflict-free for the fragment reads.
// Inside a group of 8 k's, MFMA step j of lane-half h consumes k = 4h + j for BOTH operands, which is
// what makes the two layouts interchangeable.
//
// Accumulator layout of v_mfma_f32_32x32x2_f32: register r of lane l holds
//   C[(r / 4) * 8 + (l / 32) * 4 + (r % 4)][l % 32].
#include <cstdlib>
#include <mutex>

#include "myea_device_af.h"
#include "myea_kernels.h"

namespace myea {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kThreads = 256;
constexpr int kBK = 32;
constexpr int kPadK = 4;   // k-contiguous LDS rows: BK + 4 floats (144 B, keeps 16 B alignment)
constexpr int kPadMN = 8;  // mn-contiguous LDS rows: rows + 8 floats

template <int ROWS, bool KC>
struct TileShape {
    static constexpr int kLd = KC ? (kBK + kPadK) : (ROWS + kPadMN);
    static constexpr int kFloats = KC ? ROWS * kLd : kBK * kLd;
    static constexpr int kVec = ROWS * kBK / 4;            // float4 per tile
    static constexpr int kPasses = kVec / kThreads;        // float4 per thread
    static_assert(kVec % kThreads == 0, "tile must be a multiple of the workgroup");
};

// Global -> register -> LDS mover for one operand tile (ROWS x BK): guarded scalar loads, any alignment (the general,
// slower path; aligned operands take the direct path below).
template <int ROWS, bool KC>
struct TileMover {
    using S = TileShape<ROWS, KC>;
    f32x4 reg[S::kPasses];
    const float *base; long ld; int row0, extent;

    // base: operand origin; ld: leading dimension; row0: first row (m or n) of the tile; extent: M or N
    __device__ __forceinline__ void init(const float *__restrict__ base_, long ld_, int row0_, int extent_, int)
    {
        base = base_; ld = ld_; row0 = row0_; extent = extent_;
    }

    // k0: first k of the step; K: end of the k range
    __device__ __forceinline__ void load(int k0, int K)
    {
        const int t = threadIdx.x;
#pragma unroll
        for (int p = 0; p < S::kPasses; ++p) {
            int row, k;
            if (KC) {
                constexpr int vec_per_row = kBK / 4;
                constexpr int rows_per_pass = kThreads / vec_per_row;
                row = t / vec_per_row + p * rows_per_pass;
                k = (t % vec_per_row) * 4;
            } else {
                constexpr int vec_per_k = ROWS / 4;
                constexpr int k_per_pass = kThreads / vec_per_k;
                k = t / vec_per_k + p * k_per_pass;
                row = (t % vec_per_k) * 4;
            }
            const int gr = row0 + row, gk = k0 + k;
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            if (KC) {
                const float *src = base + (long)gr * ld + gk;
                if (gr < extent) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (gk + e < K) v[e] = src[e];
                }
            } else {
                const float *src = base + (long)gk * ld + gr;
                if (gk < K) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (gr + e < extent) v[e] = src[e];
                }
            }
            reg[p] = v;
        }
    }

    __device__ __forceinline__ void fill(float *, int k0, int K) { load(k0, K); }
    __device__ __forceinline__ void commit(float *tile) const { store(tile); }
    template <int N>
    static __device__ __forceinline__ void wait() {}

    __device__ __forceinline__ void store(float *lds) const
    {
        const int t = threadIdx.x;
#pragma unroll
        for (int p = 0; p < S::kPasses; ++p) {
            int idx;
            if (KC) {
                constexpr int vec_per_row = kBK / 4;
                constexpr int rows_per_pass = kThreads / vec_per_row;
                idx = (t / vec_per_row + p * rows_per_pass) * S::kLd + (t % vec_per_row) * 4;
            } else {
                constexpr int vec_per_k = ROWS / 4;
                constexpr int k_per_pass = kThreads / vec_per_k;
                idx = (t / vec_per_k + p * k_per_pass) * S::kLd + (t % vec_per_k) * 4;
            }
            *reinterpret_cast<f32x4 *>(lds + idx) = reg[p];
        }
    }
};

// Fragment of one 32-row MFMA operand tile for a group of 8 k's: frag[j] feeds MFMA step j.
template <int ROWS, bool KC>
__device__ __forceinline__ f32x4 read_fragment(const float *lds, int tile_row, int kgroup, int lane32, int half)
{
    using S = TileShape<ROWS, KC>;
    if (KC) {
        return *reinterpret_cast<const f32x4 *>(lds + (tile_row + lane32) * S::kLd + kgroup * 8 + half * 4);
    } else {
        f32x4 v;
        const float *src = lds + (kgroup * 8 + half * 4) * S::kLd + tile_row + lane32;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = src[j * S::kLd];
        return v;
    }
}

// ---- direct global -> LDS path (16-byte aligned operands) --------------------------------------------------------
template <int ROWS, bool KC>
struct DirectShape {
    static constexpr int kPieces = ROWS * kBK * 4 / 1024;          // wavefront-wide 1 KiB pieces per tile
    static constexpr int kPerWave = kPieces / 4;
    static constexpr int kRowsPerPiece = KC ? 8 : 256 / ROWS;      // tile rows (KC) or k rows (MN) per piece
    static constexpr int kPiecePad = KC ? 0 : (ROWS == 128 ? 16 : 32);
    static constexpr int kPieceFloats = 256 + kPiecePad;
    static constexpr int kFloats = kPieces * kPieceFloats;
    static_assert(ROWS == 64 || ROWS == 128, "tile rows");
};

template <int ROWS, bool KC>
struct DirectMover {
    using S = DirectShape<ROWS, KC>;
    const float *ptr[S::kPerWave];
    int kofs[S::kPerWave];      // k of the lane's 16 bytes inside the K step (for the predicated last step)
    long step;

    __device__ __forceinline__ void init(const float *__restrict__ base, long ld, int row0, int extent, int k0)
    {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
        for (int q = 0; q < S::kPerWave; ++q) {
            const int piece = wave * S::kPerWave + q;
            if (KC) {
                const int row = piece * 8 + (lane >> 3);
                const int c = (lane & 7) ^ ((row >> 1) & 7);
                ptr[q] = base + (long)min(row0 + row, extent - 1) * ld + k0 + c * 4;
                kofs[q] = c * 4;
            } else {
                const int k = piece * S::kRowsPerPiece + (lane * 4) / ROWS, col = (lane * 4) % ROWS;
                ptr[q] = base + (long)(k0 + k) * ld + min(row0 + col, extent - 4);
                kofs[q] = k;
            }
        }
        step = KC ? (long)kBK : (long)kBK * ld;
    }

    // Starts filling `tile` (LDS) with the K step that begins at k0; K is the end of the k range.
    __device__ __forceinline__ void fill(float *tile, int k0, int K)
    {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        if (k0 + kBK <= K) {
#pragma unroll
            for (int q = 0; q < S::kPerWave; ++q) {
                float *dst = tile + (wave * S::kPerWave + q) * S::kPieceFloats;   // wave-uniform
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)ptr[q],
                                                 (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
                ptr[q] += step;
            }
        } else {   // last, partial step: through registers, zero filled along k
#pragma unroll
            for (int q = 0; q < S::kPerWave; ++q) {
                f32x4 v = {0.f, 0.f, 0.f, 0.f};
                if (k0 + kofs[q] < K) v = *reinterpret_cast<const f32x4 *>(ptr[q]);
                *reinterpret_cast<f32x4 *>(tile + (wave * S::kPerWave + q) * S::kPieceFloats + lane * 4) = v;
            }
        }
    }
    __device__ __forceinline__ void commit(float *) const {}
    // the direct loads count on vmcnt; they must have landed before the barrier that publishes the stage
    // n = number of younger loads that may stay in flight (those of the step after next)
    template <int N>
    static __device__ __forceinline__ void wait() { __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14)); }   // vmcnt(N)
};

template <int ROWS, bool KC>
__device__ __forceinline__ f32x4 read_fragment_direct(const float *lds, int tile_row, int kgroup, int lane32, int half)
{
    using S = DirectShape<ROWS, KC>;
    if (KC) {
        const int row = tile_row + lane32;
        const int slot = (kgroup * 2 + half) ^ ((row >> 1) & 7);
        return *reinterpret_cast<const f32x4 *>(lds + row * kBK + slot * 4);
    } else {
        f32x4 v;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = kgroup * 8 + half * 4 + j;
            v[j] = lds[(k / S::kRowsPerPiece) * S::kPieceFloats + (k % S::kRowsPerPiece) * ROWS + tile_row + lane32];
        }
        return v;
    }
}

// data path of one operand: how a tile gets into LDS and how fragments come out of it
template <int ROWS, bool KC, bool VEC>
struct OperandPath {
    using Mover = TileMover<ROWS, KC>;
    static constexpr int kFloats = TileShape<ROWS, KC>::kFloats;
    static constexpr int kLoads = 0;
    static __device__ __forceinline__ f32x4 frag(const float *lds, int tile_row, int g, int lane32, int half) { return read_fragment<ROWS, KC>(lds, tile_row, g, lane32, half); }
};
template <int ROWS, bool KC>
struct OperandPath<ROWS, KC, true> {
    using Mover = DirectMover<ROWS, KC>;
    static constexpr int kFloats = DirectShape<ROWS, KC>::kFloats;
    static constexpr int kLoads = DirectShape<ROWS, KC>::kPerWave;   // vmcnt events per wavefront per K step
    static __device__ __forceinline__ f32x4 frag(const float *lds, int tile_row, int g, int lane32, int half) { return read_fragment_direct<ROWS, KC>(lds, tile_row, g, lane32, half); }
};

struct GemmDev {
    const float *A, *B;
    float *C;
    int M, N, K;
    long lda, ldb, ldc;
    int accumulate, epilogue;
    const float *bias;
    float *aux_out;
    const float *colscale;
    const float *pre, *val;
    int act;
    float steep;
    const float *addend;
    long ld_addend;
    float *col_partials;
    const float *hats;
    int nbm, nbn;
    int ksplit, kchunk;   // split-K: number of slabs and k's per slab (multiple of BK); slab s writes C + s * slab
    long slab;
    float *pair_partials;    // not null: ksplit == 2 and the two workgroups of a tile combine their halves in the launch
    unsigned *pair_tickets;
    unsigned *pair_fault, *pair_host_flag;   // raised when the wait for the tile's other half runs out of polls
    unsigned pair_polls;
    int pair_local;          // the two workgroups of a tile run on one XCD (ids equal mod 8): its L2 is where they meet
};

__device__ __forceinline__ unsigned pair_xcc_id() { return __builtin_amdgcn_s_getreg(20 | (3 << 11)) & 15u; }   // HW_REG_XCC_ID[3:0]

struct TilePlace {
    int m0, n0, wave_m, wave_n, lane32, half;
    long slab_offset;
};

// The accumulators of one wavefront go out: a lane owns one column of each 32 x 32 accumulator (rows
// (r / 4) * 8 + half * 4 + r % 4), so per-column operands are read once.  The kind of epilogue, the class of the
// activation and the presence of an addend are the same for every element of a launch, and whether a tile lies wholly
// inside the matrix is the same for every element of the tile: all four are template parameters, decided once per tile,
// and the element loop carries no test of them (it carried a dozen branches per element before, 5 - 10 us per tile).
//   KIND 0 store | 3 add onto C (one hardware add per element, performed at the L2: every element is owned by exactly one
//        lane of one workgroup, so the result is the C + v a load / add / store gives, and nothing waits for C to come in)
//   KIND 1 forward: C = v + bias, aux_out = AF(C) * column multiplier; CLASS 0 no aux_out, 1 piecewise linear (linear, ReLU,
//        leaky: s < 0 ? slope * s : s, ReLU's zero kept exact), 2 through exp (sigmoid, tanh: a / (1 + exp(k s)) - b)
//   KIND 2 C = v * AF'(pre, steep, val); CLASS 1 piecewise (q < 0 ? steep * slope : steep), 2 smooth (tanh, sigmoid);
//        with col_partials, the sum of each 32-row accumulator's column goes out too: 16 values per lane, the two lanes
//        of a column combined, one store per (32-row block, column) - the bias gradient needs no pass of its own over C
// Edge tiles (WHOLE false) run the same arithmetic behind a bounds test per element, so an element's value does not
// depend on the tile shape it was computed in.
template <int KIND, int CLASS, bool ADDEND, bool WHOLE, int TM, int TN>
__device__ __forceinline__ void store_tile_as(const GemmDev &p, const f32x16 (&acc)[TM][TN], const TilePlace &at)
{
    const bool relu = p.act == MYEA_AF_RELU, tanh_like = p.act == MYEA_AF_TANH;
    const float slope = p.act == MYEA_AF_LINEAR ? 1.f : 0.01f;                       // piecewise classes (ReLU handled by `relu`)
    const float ek = tanh_like ? -2.f : -1.f, ea = tanh_like ? 2.f : 1.f, eb = tanh_like ? 1.f : 0.f;
    const float d_neg = relu ? 0.f : (p.act == MYEA_AF_LINEAR ? p.steep : p.steep * 0.01f);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int col = at.n0 + at.wave_n + j * 32 + at.lane32;
        if (!WHOLE && col >= p.N) continue;
        float bias = 0.f, cs = 1.f;
        if (KIND == 1) {
            if (p.bias) bias = p.bias[col];
            if (CLASS != 0 && p.colscale) cs = p.colscale[col];
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int row0 = at.m0 + at.wave_m + i * 32 + at.half * 4;
            float column_sum = 0.f, column_sum2 = 0.f;   // per kind: see col_partials
            // What an accumulator's elements read from other tensors - the addend, the pre-activation or the activation, x-hat -
            // is asked for four elements at a time, ahead of their arithmetic: read where it is used, every load would sit behind
            // the store of the element before it (the compiler may not move it across: the tensors could overlap) and cost its
            // own trip to memory.  (All sixteen at once need 48 more registers than the 128 x 128 tile leaves.)
#pragma unroll
            for (int rq = 0; rq < 4; ++rq) {
            float addend_v[4], operand_v[4], hats_v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = row0 + rq * 8 + e;
                addend_v[e] = 0.f; operand_v[e] = 0.f; hats_v[e] = 0.f;
                if (!WHOLE && row >= p.M) continue;
                const long o = (long)row * p.ldc + col + at.slab_offset;
                if (ADDEND) addend_v[e] = p.addend[(long)row * p.ld_addend + col];
                if (KIND == 2) {
                    operand_v[e] = CLASS == 1 ? p.pre[o] : p.val[o];
                    if (p.hats) hats_v[e] = p.hats[o];
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int r = rq * 4 + e;
                const int row = row0 + rq * 8 + e;
                if (!WHOLE && row >= p.M) continue;
                const long o = (long)row * p.ldc + col + at.slab_offset;
                float v = acc[i][j][r];
                if (ADDEND) v += addend_v[e];
                if (KIND == 1) {
                    v += bias;
                    p.C[o] = v;
                    {
#pragma clang fp contract(off)   // as for the derivative's sums below: the same bits from every tile shape
                        column_sum = column_sum + v;
                        column_sum2 = column_sum2 + v * v;
                    }
                    if (CLASS == 1) {
                        const float neg = slope * v;
                        p.aux_out[o] = (v < 0.f ? (relu ? 0.f : neg) : v) * cs;
                    } else if (CLASS == 2) {
                        const float e = expf(ek * v);
                        p.aux_out[o] = (ea / (1.f + e) - eb) * cs;
                    }
                } else if (KIND == 2) {
                    float dv;
                    if (CLASS == 1) {
                        dv = operand_v[e] < 0.f ? d_neg : p.steep;
                    } else {
                        const float y = operand_v[e];
                        dv = tanh_like ? p.steep * (1.f - y * y) : p.steep * y * (1.f - y);
                    }
                    {
#pragma clang fp contract(off)   // the sum takes the stored, rounded product - never a fused multiply-add - so every tile shape gives the same bits
                        const float out = v * dv;
                        p.C[o] = out;
                        column_sum = column_sum + out;
                        if (p.hats) column_sum2 = column_sum2 + out * hats_v[e];
                    }
                } else if (KIND == 3) {
                    unsafeAtomicAdd(&p.C[o], v);
                } else {
                    p.C[o] = v;
                }
            }
            }
            if ((KIND == 1 || KIND == 2) && p.col_partials) {
                const float both = column_sum + __shfl_xor(column_sum, 32);   // the column's other 16 rows of this accumulator
                const float both2 = column_sum2 + __shfl_xor(column_sum2, 32);
                const int block_row = at.m0 + at.wave_m + i * 32;
                if (at.half == 0 && (WHOLE || block_row < p.M)) {
                    if (KIND == 2 && !p.hats) {
                        p.col_partials[(long)(block_row >> 5) * p.N + col] = both;
                    } else {   // pairs: forward (sum, sum of squares); derivative with hats (sum of C * hats, sum of C)
                        float *pair = p.col_partials + (long)(block_row >> 5) * 2 * p.N + col;
                        pair[0] = KIND == 1 ? both : both2;
                        pair[p.N] = KIND == 1 ? both2 : both;
                    }
                }
            }
        }
    }
}

template <bool WHOLE, int TM, int TN>
__device__ __forceinline__ void store_tile_kind(const GemmDev &p, const f32x16 (&acc)[TM][TN], const TilePlace &at)
{
    const bool smooth = p.act == MYEA_AF_TANH || p.act == MYEA_AF_SIGMOID;
    if (p.epilogue == EPI_FC_FORWARD) {          // the launcher admits no addend on this kind nor on an accumulating launch
        if (!p.aux_out) store_tile_as<1, 0, false, WHOLE, TM, TN>(p, acc, at);
        else if (smooth) store_tile_as<1, 2, false, WHOLE, TM, TN>(p, acc, at);
        else store_tile_as<1, 1, false, WHOLE, TM, TN>(p, acc, at);
    } else if (p.epilogue == EPI_FC_DERIVE) {
        if (p.addend) { if (smooth) store_tile_as<2, 2, true, WHOLE, TM, TN>(p, acc, at); else store_tile_as<2, 1, true, WHOLE, TM, TN>(p, acc, at); }
        else { if (smooth) store_tile_as<2, 2, false, WHOLE, TM, TN>(p, acc, at); else store_tile_as<2, 1, false, WHOLE, TM, TN>(p, acc, at); }
    } else if (p.accumulate) {
        store_tile_as<3, 0, false, WHOLE, TM, TN>(p, acc, at);
    } else {
        if (p.addend) store_tile_as<0, 0, true, WHOLE, TM, TN>(p, acc, at);
        else store_tile_as<0, 0, false, WHOLE, TM, TN>(p, acc, at);
    }
}

// One workgroup's share of a contraction: tile number `block` of problem `p`, staged through `smem`.
template <int BM, int BN, bool A_KC, bool B_KC, bool VEC>
__device__ __forceinline__ void gemm_tile(const GemmDev &p, const int block, float *smem)
{
    constexpr int TM = BM / 64, TN = BN / 64;  // 32x32 accumulators per wavefront along m / n
    using PA = OperandPath<BM, A_KC, VEC>;
    using PB = OperandPath<BN, B_KC, VEC>;
    constexpr int kStage = PA::kFloats + PB::kFloats;  // one LDS stage = A tile then B tile

    // Workgroup -> tile.  Consecutive workgroup ids land on different XCDs (8 of them, each with its own
    // L2), so give every XCD a contiguous run of tile ids, and walk tiles in bands of 8 m-tiles so that a
    // run shares its B columns and a small set of A rows.
    const int nblocks = p.nbm * p.nbn;
    const int split = block / nblocks;   // split-K slab of this workgroup
    int pid = block - split * nblocks;
    if ((nblocks & 7) == 0) pid = (pid & 7) * (nblocks >> 3) + (pid >> 3);
    const int k_begin = split * p.kchunk, k_end = min(p.K, k_begin + p.kchunk);
    constexpr int kBand = 8;
    const int band = pid / (kBand * p.nbn);
    const int band_first = band * kBand;
    const int band_rows = min(p.nbm - band_first, kBand);
    const int in_band = pid - band * kBand * p.nbn;
    const int m0 = (band_first + in_band % band_rows) * BM;
    const int n0 = (in_band / band_rows) * BN;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lane32 = lane & 31, half = lane >> 5;
    const int wave_m = (wave >> 1) * (BM / 2), wave_n = (wave & 1) * (BN / 2);

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    typename PA::Mover moveA;
    typename PB::Mover moveB;
    const int nk = (k_end - k_begin + kBK - 1) / kBK;
    // LDS stages.  Register path: 2 (the next step's tile waits in registers).  Direct path: 3 - the loads of step
    // kt + 2 are issued while step kt computes, so a load has two steps of compute to hide behind and only the loads of
    // step kt + 1 must have landed (vmcnt(loads of one step)) at the barrier.
    constexpr int NS = (VEC && BM * BN < 128 * 128) ? 3 : 2;   // 128 x 128 keeps two stages so that two workgroups fit a CU
    constexpr int kInFlight = PA::kLoads + PB::kLoads;

    moveA.init(p.A, p.lda, m0, p.M, k_begin);
    moveB.init(p.B, p.ldb, n0, p.N, k_begin);
    moveA.fill(smem, k_begin, k_end);
    moveB.fill(smem + PA::kFloats, k_begin, k_end);
    moveA.commit(smem);
    moveB.commit(smem + PA::kFloats);
    if (NS == 3 && nk > 1) {
        moveA.fill(smem + kStage, k_begin + kBK, k_end);
        moveB.fill(smem + kStage + PA::kFloats, k_begin + kBK, k_end);
        PA::Mover::template wait<kInFlight>();
    } else {
        PA::Mover::template wait<0>();
    }
    __syncthreads();

    int cur = 0;   // stage holding step kt
    // Fragments are double buffered in registers: the LDS reads of group g + 1 are in flight while the MFMAs of group g
    // issue.  The barrier that publishes the next stage sits in front of the LAST group of a step - its fragments are
    // already in registers by then - so the first fragments of the next step are read behind that group's MFMAs
    // instead of in front of an idle matrix pipe.
    f32x4 fa[2][TM], fb[2][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[0][i] = PA::frag(smem, wave_m + i * 32, 0, lane32, half);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[0][j] = PB::frag(smem + PA::kFloats, wave_n + j * 32, 0, lane32, half);
    for (int kt = 0; kt < nk; ++kt) {
        const int ahead = NS - 1;                       // how many steps ahead the fill runs
        const bool more = kt + ahead < nk;
        int nxt = cur + ahead; if (nxt >= NS) nxt -= NS;
        float *next = smem + nxt * kStage;
        if (more) {   // that stage was last read before the previous barrier
            moveA.fill(next, k_begin + (kt + ahead) * kBK, k_end);
            moveB.fill(next + PA::kFloats, k_begin + (kt + ahead) * kBK, k_end);
        }
        const float *la = smem + cur * kStage, *lb = la + PA::kFloats;
        const int following = cur + 1 == NS ? 0 : cur + 1;   // stage of step kt + 1
#pragma unroll
        for (int g = 0; g < kBK / 8; ++g) {
            const int cb = g & 1, nb = cb ^ 1;
            if (g + 1 < kBK / 8) {
#pragma unroll
                for (int i = 0; i < TM; ++i) fa[nb][i] = PA::frag(la, wave_m + i * 32, g + 1, lane32, half);
#pragma unroll
                for (int j = 0; j < TN; ++j) fb[nb][j] = PB::frag(lb, wave_n + j * 32, g + 1, lane32, half);
            } else {
                if (more) {
                    moveA.commit(next);
                    moveB.commit(next + PA::kFloats);
                }
                // step kt + 1 must have landed; with three stages the fill of step kt + 2 may stay in flight
                if (NS == 3 && more) PA::Mover::template wait<kInFlight>();
                else PA::Mover::template wait<0>();
                __syncthreads();
                if (kt + 1 < nk) {
                    const float *na = smem + following * kStage, *nbp = na + PA::kFloats;
#pragma unroll
                    for (int i = 0; i < TM; ++i) fa[nb][i] = PA::frag(na, wave_m + i * 32, 0, lane32, half);
#pragma unroll
                    for (int j = 0; j < TN; ++j) fb[nb][j] = PB::frag(nbp, wave_n + j * 32, 0, lane32, half);
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the prefetch ahead of this group's MFMAs (the scheduler sinks it otherwise)
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cb][i][s], fb[cb][j][s], acc[i][j], 0, 0, 0);
        }
        cur = following;
    }

    if (BM == BN && p.pair_partials) {   // only launches of square tiles are split this way
        // Two workgroups share this tile, one per half of k (their ids are equal mod 8: the same XCD).  Whoever is done first
        // leaves its accumulators and goes; the other adds them and carries on to the epilogue.  The sum is half 0 + half 1
        // either way.  The wait below is for a workgroup that has nothing left to do but store its tile and raise its flag.
        __shared__ unsigned s_ticket;
        const int tile = block - split * nblocks;
        unsigned *ticket = p.pair_tickets + 2 * tile, *flag = ticket + 1;
        float *partial = p.pair_partials + (size_t)tile * (BM * BN);
        if (threadIdx.x == 0) s_ticket = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (s_ticket == 0u) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        __hip_atomic_store(partial + ((i * TN + j) * 16 + r) * kThreads + threadIdx.x, acc[i][j][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wavefront's stores are complete
            __syncthreads();
            // Publishes the tile stored above.  On one XCD the stores (performed at the L2, acknowledged) are visible to every load
            // that bypasses its compute unit's L1, and the flag carries this workgroup's XCC id for the other to check; a release
            // at device scope writes the whole L2's dirty lines back first and its acquire sends the partner's loads to memory:
            // measured 6 k + 5 k clocks against 2 k + 1.5 k.
            if (threadIdx.x == 0) {
                if (p.pair_local) __hip_atomic_store(flag, 0x100u | (pair_xcc_id() + 1u), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                else __hip_atomic_store(flag, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            }
            return;
        }
        // The wait is bounded.  When it runs out the other half is not there to add: this workgroup raises the network's fault
        // words (a device word the update kernels look at, a pinned host word the next call that looks reports) and leaves
        // without storing its tile.  Ticket and flag stay as they are - a late partner still raises its flag - and the host
        // clears both before these buffers serve another launch.
        __shared__ unsigned s_there;
        if (threadIdx.x == 0) {
            unsigned there = 0u;
            for (unsigned polls = 0; polls < p.pair_polls; ++polls) {   // plain looks; the acquire that makes the tile visible comes once, behind them
                there = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (there != 0u) break;
                __builtin_amdgcn_s_sleep(1);
            }
            // on one XCD nothing more is needed; a partner that ran elsewhere (never seen: the host probed the placement) is a fault
            if (p.pair_local && there != 0u && there != (0x100u | (pair_xcc_id() + 1u))) there = 0u;
            if (!p.pair_local && there != 0u) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
            if (there != 0u) {
                __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // as the next launch expects them
                __hip_atomic_store(flag, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
                if (p.pair_fault) __hip_atomic_store(p.pair_fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (p.pair_host_flag) __hip_atomic_store(p.pair_host_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
            s_there = there;
        }
        __syncthreads();
        if (s_there == 0u) return;
        // The other half, an accumulator at a time: its sixteen values are asked for together (device-scope loads one behind the
        // other, each used before the next was issued, cost a trip to the L2 apiece: 350 clocks x 16 x the tile's accumulators).
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                float other[16];
                if (p.pair_local) {   // served by the L2, never by this compute unit's L1
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        other[r] = __hip_atomic_load(partial + ((i * TN + j) * 16 + r) * kThreads + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                } else {
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        other[r] = __builtin_nontemporal_load(partial + ((i * TN + j) * 16 + r) * kThreads + threadIdx.x);
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = split == 0 ? acc[i][j][r] + other[r] : other[r] + acc[i][j][r];
            }
    }
    // Epilogue.  What kind it is, whether an addend joins and whether the tile lies wholly inside the matrix are the same
    // for every element of the tile: they are decided once, and the element loops of whole tiles carry no such test.
    const TilePlace at{m0, n0, wave_m, wave_n, lane32, half, (long)split * p.slab};
    if (m0 + BM <= p.M && n0 + BN <= p.N) store_tile_kind<true, TM, TN>(p, acc, at);
    else store_tile_kind<false, TM, TN>(p, acc, at);
}

template <int BM, int BN, bool A_KC, bool B_KC, bool VEC>
__global__ __launch_bounds__(kThreads, 2) void gemm_f32_mfma_kernel(GemmDev p)
{
    extern __shared__ __attribute__((aligned(16))) float smem[];
    gemm_tile<BM, BN, A_KC, B_KC, VEC>(p, (int)blockIdx.x, smem);
}

// Two independent contractions in one launch, 128 x 128 tiles each: workgroups [0, first_blocks) work on `a` (A k-contiguous,
// B n-contiguous: dX = delta W), the others on `b` (both operands k-strided: dW += delta^T X).  A batch of 1024 gives dX only
// 256 such tiles - one workgroup per CU, one wavefront per SIMD, too little to keep the matrix pipe busy - while dW has
// four times as many, quarter as long.  Launched together, a CU holds one long dX workgroup next to a succession of
// dW workgroups: two wavefronts per SIMD throughout, and the dW tiles' stores fall at different moments behind
// the dX workgroup's MFMAs instead of all at once.
// At a batch of 512 the same holds one size down: dX as 64 x 64 tiles (256 of them for 2048-wide layers) beside dW as
// 128 x 128 tiles over the short k = batch, equal work per workgroup, one of each per CU.
template <int BMA, int BNA>
__global__ __launch_bounds__(kThreads, 2) void gemm_pair_kernel(GemmDev a, GemmDev b, int first_blocks)
{
    extern __shared__ __attribute__((aligned(16))) float smem[];
    if ((int)blockIdx.x < first_blocks) gemm_tile<BMA, BNA, true, false, true>(a, (int)blockIdx.x, smem);
    else gemm_tile<128, 128, false, false, true>(b, (int)blockIdx.x - first_blocks, smem);
}

template <int BM, int BN, bool A_KC, bool B_KC, bool VEC>
int launch_one(hipStream_t stream, GemmDev d)
{
    constexpr size_t lds_bytes = ((VEC && BM * BN < 128 * 128) ? 3 : 2) * (OperandPath<BM, A_KC, VEC>::kFloats + OperandPath<BN, B_KC, VEC>::kFloats) * sizeof(float);
    auto kern = gemm_f32_mfma_kernel<BM, BN, A_KC, B_KC, VEC>;
    static std::once_flag attr_once;  // per instantiation; launches may come from several host threads
    static hipError_t attr_status = hipSuccess;
    std::call_once(attr_once, [&] { attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes); });
    if (attr_status != hipSuccess) return hip_fail(attr_status, "hipFuncSetAttribute(gemm_f32_mfma_kernel)");
    d.nbm = (d.M + BM - 1) / BM;
    d.nbn = (d.N + BN - 1) / BN;
    const long nblocks = (long)d.nbm * d.nbn * d.ksplit;
    if (nblocks <= 0 || nblocks > 0x7fffffffL) { set_last_error("gemm: grid of %ld workgroups out of range", nblocks); return MYEA_E_INVALID; }
    hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(kThreads), lds_bytes, stream, d);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

template <int BM, int BN>
int launch_layout_vec(hipStream_t stream, const GemmDev &d, bool a_kc, bool b_kc)
{
    if (a_kc && b_kc) return launch_one<BM, BN, true, true, true>(stream, d);
    if (a_kc && !b_kc) return launch_one<BM, BN, true, false, true>(stream, d);
    return launch_one<BM, BN, false, false, true>(stream, d);
}

// short-M, short-N problems (the per-time-step recurrent contractions): 64 x 64 tiles
int launch_layout_vec_small(hipStream_t stream, const GemmDev &d, bool a_kc, bool b_kc)
{
    if (a_kc && b_kc) return launch_one<64, 64, true, true, true>(stream, d);
    if (a_kc && !b_kc) return launch_one<64, 64, true, false, true>(stream, d);
    return launch_one<64, 64, false, false, true>(stream, d);
}

// guarded scalar loads, any alignment, any layout: the general (slow) path
int launch_layout_scalar(hipStream_t stream, const GemmDev &d, bool a_kc, bool b_kc)
{
    if (a_kc && b_kc) return launch_one<64, 64, true, true, false>(stream, d);
    if (a_kc && !b_kc) return launch_one<64, 64, true, false, false>(stream, d);
    if (!a_kc && !b_kc) return launch_one<64, 64, false, false, false>(stream, d);
    return launch_one<64, 64, false, true, false>(stream, d);
}


// ---- a narrow product ---------------------------------------------------------------------------------------------------
// C [M][N] = A B with N <= 32 and K <= 64 - a layer of an independently recurrent stack over T x batch rows, forward or backward.
// The tiled kernel spends such a launch on its set-up, its predicated scalar loads and its stages (rows of 31 floats are no
// 16-byte multiples): a few microseconds of instructions fetched to be run once.  Here a wavefront owns 32 rows of C: the
// lane's operands of v_mfma_f32_32x32x2f32 are asked for straight from memory, all of a round of 32 k's together (A: lane l
// takes row l % 32 at k + l / 32; B: column l % 32), then the round's 16 matrix instructions; no LDS, one round or two.  The
// accumulator has the layout of the tiled kernel's, so its epilogue (store_tile_kind) finishes the tile: every kind of
// epilogue, the same arithmetic per element.
template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(kThreads) void narrow_gemm_kernel(GemmDev p)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, lane32 = lane & 31, half = lane >> 5;
    const int m0 = (int)blockIdx.x * 128, row = m0 + wave * 32 + lane32;
    const bool in_m = row < p.M, in_n = lane32 < p.N;
    f32x16 acc[1][1];
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[0][0][r] = 0.f;
    const float *a_at = A_KC ? p.A + (long)row * p.lda + half : p.A + (long)half * p.lda + row;
    const float *b_at = B_KC ? p.B + (long)lane32 * p.ldb + half : p.B + (long)half * p.ldb + lane32;
    const long a_step = A_KC ? 2 : 2 * p.lda, b_step = B_KC ? 2 : 2 * p.ldb;   // from one pair of k's to the next
    for (int k0 = 0; k0 < p.K; k0 += 32) {
        float a[16], b[16];
#pragma unroll
        for (int s = 0; s < 16; ++s) {
            const bool in_k = k0 + 2 * s + half < p.K;
            a[s] = (in_m && in_k) ? a_at[s * a_step] : 0.f;
            b[s] = (in_n && in_k) ? b_at[s * b_step] : 0.f;
        }
#pragma unroll
        for (int s = 0; s < 16; ++s) acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[s], acc[0][0], 0, 0, 0);
        a_at += 16 * a_step; b_at += 16 * b_step;
    }
    const TilePlace at{m0, 0, wave * 32, 0, lane32, half, 0L};
    if (m0 + 128 <= p.M && p.N == 32) store_tile_kind<true, 1, 1>(p, acc, at);
    else store_tile_kind<false, 1, 1>(p, acc, at);
}

// ---- the weight gradient of a narrow layer ------------------------------------------------------------------------------
// dW = delta^T X with at most 32 outputs (columns of delta) and at most 32 inputs (columns of X) over many rows - a layer of an
// independently recurrent stack over T x batch rows.  Two rows of delta and of X, as they lie in memory, ARE the operands of
// v_mfma_f32_32x32x2f32 (lane l: column l % 32 of row l / 32): a wavefront walks its share of the rows with two coalesced
// loads and one matrix instruction per pair of rows, no LDS, no tile edges to test; a loop of a few dozen instructions.
// The wavefronts of a workgroup add their 32 x 32 accumulators in wavefront order and store one slab [H][In]; the slabs
// are added by launch_slab_sum_add, as the slabs of a split-K launch are.  (The tiled kernel spends its time on such a
// shape in its set-up, its predicated scalar loads of operands whose rows are not 16-byte multiples, and its epilogue.)
constexpr int kNarrowAhead = 16;   // pairs of rows a wavefront asks for at once: its whole share when the launch is not capped
constexpr int kNarrowWaves = 8;    // wavefronts a workgroup: fewer slabs to add afterwards
__global__ __launch_bounds__(64 * kNarrowWaves) void narrow_dw_kernel(const float *__restrict__ delta, const float *__restrict__ x, float *__restrict__ slabs,
                                                             int H, int In, long rows, long rows_per_wave)
{
    __shared__ float handed[kNarrowWaves - 1][16][64];   // the accumulators of the wavefronts behind the first
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 31, half = lane >> 5;
    const long first = ((long)blockIdx.x * kNarrowWaves + wave) * rows_per_wave;
    const long last = first + rows_per_wave < rows ? first + rows_per_wave : rows;
    const bool in_delta = col < H, in_x = col < In;
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    for (long r0 = first; r0 < last; r0 += 2 * kNarrowAhead) {
        float a[kNarrowAhead], b[kNarrowAhead];
#pragma unroll
        for (int u = 0; u < kNarrowAhead; ++u) {
            const long row = r0 + 2 * u + half;
            a[u] = (in_delta && row < last) ? delta[row * H + col] : 0.f;
            b[u] = (in_x && row < last) ? x[row * In + col] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < kNarrowAhead; ++u) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[u], acc, 0, 0, 0);
    }
    if (wave) {
#pragma unroll
        for (int r = 0; r < 16; ++r) handed[wave - 1][r][lane] = acc[r];
    }
    __syncthreads();
    if (wave || !in_x) return;
    float *slab = slabs + (size_t)blockIdx.x * H * In;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int m = (r >> 2) * 8 + half * 4 + (r & 3);   // the accumulator's row of this lane's column
        float v = acc[r];
#pragma unroll
        for (int w = 0; w < kNarrowWaves - 1; ++w) v += handed[w][r][lane];
        if (m < H) slab[m * In + col] = v;
    }
}

}  // namespace

// Number of K slabs for a contraction whose M x N alone does not fill the chip; 1 when the plain launch already does.
// Short k: about one workgroup per CU with 64 x 64 tiles, each slab at least 128 k's deep.
int gemm_split_k(int M, int N, int K)
{
    const long tiles_128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    if (tiles_128 * 2 >= 256) return 1;
    long want;
    if (K >= 4096) {
        // long k (weight gradients over T x batch rows): enough slabs for ~1000 workgroups of 128 x 64, each slab at least
        // 1024 k's deep - the larger tile's operand reuse is worth more than the pass over the slabs that sums them
        want = (512 + tiles_128 - 1) / tiles_128;
        // (a product no larger than one 64 x 64 tile has no operand reuse to protect: slabs 256 k's deep, up to 32 of them)
        const long depth = (M <= 64 && N <= 64) ? 256 : 1024;
        if (want > K / depth) want = K / depth;
        if (depth == 256) { if (want > 32) want = 32; if (want < 1) want = 1; const int c = (int)(((K + want - 1) / want + kBK - 1) / kBK * kBK); return (K + c - 1) / c; }
    } else {
        const long tiles_64 = (long)((M + 63) / 64) * ((N + 63) / 64);
        want = (256 + tiles_64 - 1) / tiles_64;
        const long max_by_k = K / 128 > 0 ? K / 128 : 1;
        if (want > max_by_k) want = max_by_k;
    }
    if (want > 16) want = 16;
    if (want < 1) want = 1;
    // the launcher rounds the chunk up to a multiple of 32: return the slab count that rounding produces
    const int chunk = (int)(((K + want - 1) / want + kBK - 1) / kBK * kBK);
    return (K + chunk - 1) / chunk;
}

unsigned gemm_pair_polls()
{
    const char *e = std::getenv("MYEA_GEMM_PAIR_SPIN_POLLS");
    if (e && *e) { const unsigned long long v = std::strtoull(e, nullptr, 10); return v > 0xffffffffull ? 0xffffffffu : (unsigned)v; }
    return 1u << 24;
}

bool gemm_pair_k_128(int M, int N, int K)
{
    const long tiles_128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    return tiles_128 <= kGemmPairTiles && tiles_128 % 8 == 0 && tiles_128 >= 128 && K >= 2048;
}

bool gemm_can_fuse_activation(int act)
{
    return act == MYEA_AF_LINEAR || act == MYEA_AF_RELU || act == MYEA_AF_LEAKY_RELU || act == MYEA_AF_PARAMETRIC_RELU ||
           act == MYEA_AF_TANH || act == MYEA_AF_SIGMOID;
}

// checks a problem and fills the kernel's argument block; *vec: operands take the direct (16-byte aligned) path
static int prepare_gemm(const GemmParams &p, GemmDev &d, bool *vec)
{
    if (p.M <= 0 || p.N <= 0 || p.K < 0) { set_last_error("gemm: bad shape M=%d N=%d K=%d", p.M, p.N, p.K); return MYEA_E_INVALID; }
    if (!p.A || !p.B || !p.C) { set_last_error("gemm: null operand"); return MYEA_E_INVALID; }
    const long a_min = p.a_k_contiguous ? p.K : p.M, b_min = p.b_k_contiguous ? p.K : p.N;
    if (p.lda < a_min || p.ldb < b_min || p.ldc < p.N) { set_last_error("gemm: leading dimension smaller than the row length"); return MYEA_E_INVALID; }
    if (p.epilogue == EPI_FC_DERIVE && (!p.pre || !p.val)) { set_last_error("gemm: derive epilogue without pre/val"); return MYEA_E_INVALID; }
    if (p.addend && (p.epilogue == EPI_FC_FORWARD || p.accumulate)) { set_last_error("gemm: an addend goes with a plain or a derivative epilogue only"); return MYEA_E_INVALID; }
    if (p.epilogue == EPI_FC_DERIVE && !gemm_can_fuse_activation(p.act)) { set_last_error("gemm: activation %d cannot be fused", p.act); return MYEA_E_INVALID; }
    if (p.epilogue == EPI_FC_FORWARD && p.aux_out && !gemm_can_fuse_activation(p.act)) { set_last_error("gemm: activation %d cannot be fused", p.act); return MYEA_E_INVALID; }

    d.A = p.A; d.B = p.B; d.C = p.C;
    d.M = p.M; d.N = p.N; d.K = p.K;
    d.lda = p.lda; d.ldb = p.ldb; d.ldc = p.ldc;
    d.accumulate = (p.accumulate && !p.c_is_zero) ? 1 : 0; d.epilogue = p.epilogue;   // onto zeros a store gives the same values as an add
    d.bias = p.bias; d.aux_out = p.aux_out; d.colscale = p.colscale;
    d.pre = p.pre; d.val = p.val; d.act = p.act; d.steep = p.steep;
    d.addend = p.addend; d.ld_addend = p.ld_addend;
    d.col_partials = p.col_partials; d.hats = p.hats;
    if (p.col_partials && p.epilogue == EPI_NONE) { set_last_error("gemm: column partial sums go with the forward and the derivative epilogue only"); return MYEA_E_INVALID; }
    if (p.hats && (p.epilogue != EPI_FC_DERIVE || !p.col_partials)) { set_last_error("gemm: hats go with the derivative epilogue's column sums"); return MYEA_E_INVALID; }
    if (p.addend && (p.epilogue == EPI_FC_FORWARD || p.ld_addend < p.N)) { set_last_error("gemm: addend needs EPI_NONE / EPI_FC_DERIVE and ld_addend >= N"); return MYEA_E_INVALID; }
    d.nbm = d.nbn = 0;
    d.ksplit = 1; d.kchunk = p.K > 0 ? p.K : 1; d.slab = 0;
    d.pair_partials = nullptr; d.pair_tickets = nullptr;
    d.pair_fault = p.pair_fault; d.pair_host_flag = p.pair_host_flag; d.pair_polls = p.pair_polls;
    {   // MYEA_GEMM_PAIR_LOCAL=0: the two workgroups of a tile meet through device-scope release / acquire wherever they run
        static const bool local_off = [] { const char *e = std::getenv("MYEA_GEMM_PAIR_LOCAL"); return e && e[0] == '0'; }();
        d.pair_local = (!local_off && device_groups_share_xcd()) ? 1 : 0;
    }
    if (p.split_k > 1) {
        if (p.epilogue != EPI_NONE || p.accumulate || p.addend) { set_last_error("gemm: split-K writes plain partial slabs"); return MYEA_E_INVALID; }
        const int chunk = ((p.K + p.split_k - 1) / p.split_k + kBK - 1) / kBK * kBK;
        d.kchunk = chunk;
        d.ksplit = (p.K + chunk - 1) / chunk;
        d.slab = p.split_k_slab;
        if (d.ksplit != p.split_k) { set_last_error("gemm: split-K count %d does not divide K=%d into %d-wide chunks; use gemm_split_k()", p.split_k, p.K, chunk); return MYEA_E_INVALID; }
    }

    // 128-bit global loads need 16-byte aligned rows; otherwise fall back to guarded scalar loads.
    auto aligned = [](const float *ptr, long ld, long contiguous_extent) {
        return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0 && (ld & 3) == 0 && (contiguous_extent & 3) == 0;
    };
    *vec = aligned(p.A, p.lda, p.a_k_contiguous ? p.K : p.M) && aligned(p.B, p.ldb, p.b_k_contiguous ? p.K : p.N);
    return MYEA_OK;
}

// Slabs the narrow weight-gradient kernel writes for these shapes: 0 when the shape is not its own (the tiled kernel takes it).
// A wavefront gets at least 32 rows (one round of loads), a launch at most 128 workgroups.
int narrow_dw_slabs(size_t H, size_t In, size_t rows)
{
    if (H == 0 || In == 0 || H > 32 || In > 32 || rows < 512 || rows > 0x7fffffffu) return 0;
    static const bool off = [] { const char *e = std::getenv("MYEA_NARROW_DW"); return e && e[0] == '0'; }();
    if (off) return 0;
    size_t per_wave = 2 * kNarrowAhead;
    while ((rows + kNarrowWaves * per_wave - 1) / (kNarrowWaves * per_wave) > 128) per_wave *= 2;
    return (int)((rows + kNarrowWaves * per_wave - 1) / (kNarrowWaves * per_wave));
}

// delta [rows][H], x [rows][In], both dense; slabs: narrow_dw_slabs(H, In, rows) x [H][In]
int launch_narrow_dw(hipStream_t stream, const float *delta, const float *x, float *slabs, size_t H, size_t In, size_t rows)
{
    const int S = narrow_dw_slabs(H, In, rows);
    if (S <= 0 || !delta || !x || !slabs) { set_last_error("narrow weight gradient: %zu x %zu over %zu rows is not its shape", H, In, rows); return MYEA_E_INVALID; }
    const long per_wave = (long)(((rows + (size_t)S * kNarrowWaves - 1) / ((size_t)S * kNarrowWaves) + 1) / 2 * 2);   // even: a matrix instruction takes a pair of rows
    hipLaunchKernelGGL(narrow_dw_kernel, dim3((unsigned)S), dim3(64 * kNarrowWaves), 0, stream, delta, x, slabs, (int)H, (int)In, (long)rows, per_wave);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

int launch_gemm(hipStream_t stream, const GemmParams &p)
{
    GemmDev d;
    bool vec = false;
    {
        const int rc = prepare_gemm(p, d, &vec);
        if (rc != MYEA_OK) return rc;
    }
    const bool a_kc = p.a_k_contiguous != 0, b_kc = p.b_k_contiguous != 0;

    // a narrow product over many rows: the kernel that feeds the matrix unit straight from memory (MYEA_NARROW_GEMM=0: the tiled one)
    static const bool narrow_off = [] { const char *e = std::getenv("MYEA_NARROW_GEMM"); return e && e[0] == '0'; }();
    if (!narrow_off && p.N <= 32 && p.K <= 64 && p.M >= 256 && d.ksplit == 1) {
        const dim3 grid((unsigned)((p.M + 127) / 128));
        if (a_kc && b_kc) hipLaunchKernelGGL((narrow_gemm_kernel<true, true>), grid, dim3(kThreads), 0, stream, d);
        else if (a_kc) hipLaunchKernelGGL((narrow_gemm_kernel<true, false>), grid, dim3(kThreads), 0, stream, d);
        else if (b_kc) hipLaunchKernelGGL((narrow_gemm_kernel<false, true>), grid, dim3(kThreads), 0, stream, d);
        else hipLaunchKernelGGL((narrow_gemm_kernel<false, false>), grid, dim3(kThreads), 0, stream, d);
        MYEA_HIP_TRY(hipGetLastError());
        return MYEA_OK;
    }
    if (!vec || (!a_kc && b_kc)) return launch_layout_scalar(stream, d, a_kc, b_kc);
    // Tile choice: 128 x 128 when that still yields at least two workgroups per CU (256 CUs), else
    // 64-row tiles to keep the chip filled for short-M / short-N problems.
    const long tiles_128 = (long)((p.M + 127) / 128) * ((p.N + 127) / 128);
    if (tiles_128 * d.ksplit >= 512) return launch_layout_vec<128, 128>(stream, d, a_kc, b_kc);   // slabs of a split k count: they fill the chip like tiles do
    // At most one 64 x 64 tile per compute unit and a k worth splitting: two workgroups per tile, half of k each, combined in
    // the launch - a second wavefront per SIMD to fill the first one's waits, which such a launch otherwise lacks.
    // MYEA_GEMM_PAIR_K=0 keeps one workgroup per tile.
    static const int pair_k = [] { const char *e = std::getenv("MYEA_GEMM_PAIR_K"); return e ? std::atoi(e) : 3; }();   // bit 0: 64 x 64 tiles, bit 1: 128 x 128
    const bool pair_k_off = !(pair_k & 1);
    // The same one size up: at most one 128 x 128 tile per compute unit (a batch of 1024 in front of 4096 units) would run as 64 x
    // 128 tiles to put two workgroups on every compute unit; two workgroups sharing a 128 x 128 tile's k do that with the larger
    // tile's operand reuse.
    if ((pair_k & 2) && p.pair_partials && p.pair_tickets && d.ksplit == 1 && gemm_pair_k_128(p.M, p.N, p.K)) {
        d.ksplit = 2;
        d.kchunk = ((p.K + 1) / 2 + kBK - 1) / kBK * kBK;
        d.pair_partials = p.pair_partials; d.pair_tickets = p.pair_tickets;
        return launch_layout_vec<128, 128>(stream, d, a_kc, b_kc);
    }
    const long tiles_64 = (long)((p.M + 63) / 64) * ((p.N + 63) / 64);
    if (p.pair_partials && p.pair_tickets && !pair_k_off && d.ksplit == 1 && tiles_64 <= kGemmPairTiles && tiles_64 % 8 == 0 && tiles_64 >= 128 && p.K >= 512) {
        d.ksplit = 2;
        d.kchunk = ((p.K + 1) / 2 + kBK - 1) / kBK * kBK;
        d.pair_partials = p.pair_partials; d.pair_tickets = p.pair_tickets;
        return launch_layout_vec_small(stream, d, a_kc, b_kc);
    }
    if (tiles_128 * 2 * d.ksplit < 256) return launch_layout_vec_small(stream, d, a_kc, b_kc);
    if (p.M <= p.N) return launch_layout_vec<64, 128>(stream, d, a_kc, b_kc);
    return launch_layout_vec<128, 64>(stream, d, a_kc, b_kc);
}

// `a` = (A k-contiguous, B n-contiguous), `b` = (both k-strided), neither split along k, 16-byte aligned operands, and `a`
// no more than about one 128 x 128 tile per CU: both in ONE launch (gemm_pair_kernel).  Returns MYEA_OK when launched,
// 1 when the pair form does not apply (the caller launches the two one after the other), a negative code on an error.
int launch_gemm_pair(hipStream_t stream, const GemmParams &a, const GemmParams &b)
{
    if (!a.a_k_contiguous || a.b_k_contiguous || b.a_k_contiguous || b.b_k_contiguous || a.split_k > 1 || b.split_k > 1) return 1;
    GemmDev da, db;
    bool va = false, vb = false;
    int rc = prepare_gemm(a, da, &va);
    if (rc != MYEA_OK) return rc;
    rc = prepare_gemm(b, db, &vb);
    if (rc != MYEA_OK) return rc;
    if (!va || !vb) return 1;
    db.nbm = (b.M + 127) / 128; db.nbn = (b.N + 127) / 128;
    const long nb = (long)db.nbm * db.nbn;
    // Worth it when `a` alone would leave the CUs with one workgroup each and `b` brings about as much work in at least as
    // many pieces: `a` as 128 x 128 tiles if that gives 128 .. 256 of them, else as 64 x 64 tiles under the same test.
    auto fits = [&](int tile) {
        const long na = (long)((a.M + tile - 1) / tile) * ((a.N + tile - 1) / tile);
        const double wa = (double)a.K * tile * tile * (double)na, wb = (double)b.K * 128.0 * 128.0 * (double)nb;
        return na >= 128 && na <= 256 && (na & 7) == 0 && nb >= na && wa <= 2.0 * wb && wb <= 2.0 * wa;
    };
    constexpr size_t lds_b = 2 * (OperandPath<128, false, true>::kFloats + OperandPath<128, false, true>::kFloats) * sizeof(float);
    if (fits(128)) {
        // beside a long dX of 128 x 128 tiles the adds at the L2 were measured faster than stores (4096-wide layers at batch
        // 1024: 475 against 482 us); everywhere else a store onto known zeros wins
        static const int store128 = [] { const char *e = std::getenv("MYEA_DW_STORE_PAIR128"); return e ? std::atoi(e) : 0; }();
        if (b.accumulate && !store128) db.accumulate = 1;
        da.nbm = (a.M + 127) / 128; da.nbn = (a.N + 127) / 128;
        const long na = (long)da.nbm * da.nbn;
        constexpr size_t lds_a = 2 * (OperandPath<128, true, true>::kFloats + OperandPath<128, false, true>::kFloats) * sizeof(float);
        constexpr size_t lds_bytes = lds_a > lds_b ? lds_a : lds_b;
        static std::once_flag attr_once;
        static hipError_t attr_status = hipSuccess;
        std::call_once(attr_once, [&] { attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_pair_kernel<128, 128>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes); });
        if (attr_status != hipSuccess) return hip_fail(attr_status, "hipFuncSetAttribute(gemm_pair_kernel)");
        hipLaunchKernelGGL((gemm_pair_kernel<128, 128>), dim3((unsigned)(na + nb)), dim3(kThreads), lds_bytes, stream, da, db, (int)na);
    } else if (fits(64)) {
        da.nbm = (a.M + 63) / 64; da.nbn = (a.N + 63) / 64;
        const long na = (long)da.nbm * da.nbn;
        constexpr size_t lds_a = 3 * (OperandPath<64, true, true>::kFloats + OperandPath<64, false, true>::kFloats) * sizeof(float);
        constexpr size_t lds_bytes = lds_a > lds_b ? lds_a : lds_b;
        static std::once_flag attr_once;
        static hipError_t attr_status = hipSuccess;
        std::call_once(attr_once, [&] { attr_status = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_pair_kernel<64, 64>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes); });
        if (attr_status != hipSuccess) return hip_fail(attr_status, "hipFuncSetAttribute(gemm_pair_kernel)");
        hipLaunchKernelGGL((gemm_pair_kernel<64, 64>), dim3((unsigned)(na + nb)), dim3(kThreads), lds_bytes, stream, da, db, (int)na);
    } else {
        return 1;
    }
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

}  // namespace myea

extern "C" int myea_hip_gemm_f32(void *stream, int a_k_contiguous, int b_k_contiguous, int accumulate, size_t M, size_t N, size_t K,
                                 const float *A, size_t lda, const float *B, size_t ldb, float *C, size_t ldc)
{
    if (M > 0x7fffffffu || N > 0x7fffffffu || K > 0x7fffffffu) { myea::set_last_error("gemm: dimension too large"); return MYEA_E_INVALID; }
    myea::GemmParams p{};
    p.A = A; p.B = B; p.C = C;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    p.lda = (long)lda; p.ldb = (long)ldb; p.ldc = (long)ldc;
    p.a_k_contiguous = a_k_contiguous; p.b_k_contiguous = b_k_contiguous;
    p.accumulate = accumulate;
    p.epilogue = myea::EPI_NONE;
    return myea::launch_gemm(static_cast<hipStream_t>(stream), p);
}
