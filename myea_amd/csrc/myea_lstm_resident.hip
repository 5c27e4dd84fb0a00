// myea_lstm_resident.hip — the time loop of an LSTM layer as ONE launch: a workgroup stays on its compute unit for all
// time steps, keeps its slice of the recurrent weights in registers, and meets the other workgroups that share its
// examples at a bounded barrier between steps.
//
// Why: as one launch per time step (myea_lstm_fused.hip) every step pays a launch, the fill and drain of a kernel that
// lives for 10 us, and a fresh fetch of the workgroup's 128 KB weight slice.  The recurrence only needs, per step, what
// the previous step produced for the SAME examples: workgroups that own different examples never talk.
//
// Shape of the work (one cell per block, C cells, gate rows z | i | f | o of the packed matrices):
//   * a workgroup owns CELLS cells (16, or 8 when C > 512).  Forward: the 4 CELLS gate columns of those cells, its four wavefronts split
//     k = C into contiguous quarters; backward: the CELLS columns of dh, wavefront w takes the k range of gate w.  Either
//     way a wavefront holds its [columns][k range] slice of Wrec (WrecT) in registers for the whole launch (at most 128
//     registers per lane) in the operand layout of v_mfma_f32_16x16x4_f32.  The backward loop has a second form, split
//     along k instead of along the columns (described at its kernel), which is the one taken when the layer leaves half of
//     the compute units or more idle;
//   * a GROUP is the set of workgroups that cover all C cells for 2 x ROWS examples of one direction (ROWS = 16 RS):
//     C / CELLS members.  A member is a workgroup of four wavefronts - one per SIMD - that lives for all T steps and keeps
//     its slice of the recurrent matrix in registers.  It works on two independent CHAINS of ROWS examples in turn: a
//     UNIT is one time step of one chain, and the units of the two chains alternate in program order.
//   * A unit: the exchanged tensor of the chain's examples (h[t-1] forward, the gate deltas dG[t+1] backward) arrives in
//     LDS (global -> LDS directly, every wavefront only its own k range); MFMAs against the register-resident weights; the
//     four partial tiles meet in LDS; gate math of the lane's (example, cell) pair(s); stores.
//   * On this device the fp32 MFMAs and ordinary vector instructions of a SIMD do not overlap, whichever wavefront they
//     come from (measured), so a second wavefront per SIMD buys no issue slots; what can be hidden is latency.  (The 512-cell
//     backward loop does give each chain its own set of four wavefronts - lstm_resident_backward_sets_kernel - because its
//     tail is mostly latency: described there.)  In one instruction stream the chain that is not computing is the one whose
//     stores, barrier and tile loads are in flight:
//       - a unit's arrival at its chain's counter is signalled a quarter into the NEXT unit's MFMAs, when its stores have
//         long been acknowledged;
//       - the counter is read three quarters into those MFMAs and is normally complete at their end;
//       - the tiles of the unit after that are requested then, and land under the partial exchange and the gate math.
//
// Barriers and visibility.  Two protocols, chosen on the host:
//   * LOCAL: every member of a group runs on the same XCD (workgroup ids that are equal mod 8 share an XCD; the host
//     checks that with a probe launch once per process, and in every launch the members of a group compare their XCC
//     ids).  The XCD's L2 is then the point of coherence: plain stores, a counter bumped by an atomic performed in L2 and
//     polled with loads that bypass the compute unit's L1 (sc1), as do the loads of the exchanged tensor;
//   * AGENT (groups wider than an XCD, C = 1024, forward only): device-scope stores of h, device-scope counter, sc1 loads.
// A wavefront arrives once its own stores are complete (vmcnt(0)); the last of the four - counted in LDS - bumps the
// chain's counter.  A wait is bounded: after `spin_polls` polls the waiting wavefront raises the give-up flag, every
// wavefront sees it at its next poll and leaves, the kernel ends normally and the host reports MYEA_E_DEVICE.
// The host only launches when every workgroup of the grid can be resident at once (one per compute unit).
//
// vmcnt: the loads and stores of a wavefront complete in issue order as far as the counter is concerned, so "at most N
// outstanding" with N = the stores issued after a unit's tile loads says that the tiles have landed.  Every lane issues
// the same stores: lanes whose example lies beyond the batch write to a scrap area.
//
// Gate math: Forward_Pass__LSTM__Gates_CIF_AF_State (NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:1042-1191),
// __States_AF (:1547-1582), __Output (:1351-1418); backward: Backward_Pass__LSTM_Derivative__Output
// (NN/Neural_Network__Recurrent_Backward_Pass__OpenMP.cpp:1130-1273), __Cell_State_AF (:1275-1327),
// __Gates_CIF_AF_State (:1329-1604).  NN/ = Neural_Network_Library_Windows/Source_Files/Neural_Network/.
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <type_traits>
#include <vector>

#include "myea_kernels.h"

namespace myea {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;      // four wavefronts, one per SIMD
constexpr int kSyncStride = 32;    // counters sit 128 bytes apart
constexpr int kMaxGroups = 64;     // groups a network's counter block holds
constexpr int kScrapWords = 8192;   // where lanes without an example put their stores: 4 gate rows of up to 1024 + 4 x 1024
constexpr int kLocalAux = 16;      // cache policy of the LOCAL protocol's tile loads: sc1, served by L2, never by this compute unit's L1

#define MYEA_SCOPE_AGENT __HIP_MEMORY_SCOPE_AGENT
#define MYEA_SCOPE_WORKGROUP __HIP_MEMORY_SCOPE_WORKGROUP

// LDS of a workgroup: every wavefront's tiles of one unit, and the partial tiles of the two chains
constexpr size_t forward_lds(int kw, int cells, int rs) { return ((size_t)4 * (kw / 32) * 16 * rs * 32 + (size_t)2 * 4 * 16 * rs * (4 * cells + 8)) * sizeof(float); }
constexpr size_t backward_sets_lds(int c) { return ((size_t)8 * (c / 32 < 8 ? c / 32 : 8) * 16 * 32 + (size_t)2 * 4 * 16 * 17) * sizeof(float); }
constexpr size_t backward_lds(int c, int rs) { return ((size_t)4 * (c >= 512 && rs == 1 ? c / 64 : c / 32) * 16 * rs * 32 + (size_t)2 * 4 * 16 * rs * 17) * sizeof(float); }

template <int N>
__device__ __forceinline__ void wait_vm() { __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14)); }   // vmcnt(N)

// Workgroup barrier for data exchanged through LDS only: waits for this wavefront's LDS operations, not for its global
// loads and stores (the next unit's tiles are in flight across it).
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
}

// exp2 and reciprocal instructions (1 ulp each) instead of the library's expf and an IEEE division: the error stays some
// orders of magnitude below the tolerance the gate activations are held to, and the vector pipe is what a unit waits for
__device__ __forceinline__ float sigmoid_f(float s) { return __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.44269504088896341f * s)); }
__device__ __forceinline__ float tanh_f(float s) { return 2.f * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-2.88539008177792681f * s)) - 1.f; }  // AF_TANH_real

// [ROWS][32 k] tile of one wavefront in LDS, 16-byte chunks XOR-swizzled by (row >> 1) & 7; one direct load brings 8 rows.
// AUX = 16 (sc1): the load is served beyond this compute unit's L1 at device scope; AUX = 0: a plain load.
template <int ROWS, int AUX>
struct ATile {
    const float *ptr[ROWS / 8];
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
    // tile number `i` of the wavefront's k range
    __device__ __forceinline__ void fill(float *tile, int i) const
    {
#pragma unroll
        for (int q = 0; q < ROWS / 8; ++q)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(ptr[q] + i * 32),
                                             (__attribute__((address_space(3))) void *)(tile + q * 256), 16, 0, AUX);
    }
    static __device__ __forceinline__ f32x4 chunk(const float *tile, int row, int c)
    {
        return *reinterpret_cast<const f32x4 *>(tile + row * 32 + ((c ^ ((row >> 1) & 7)) << 2));
    }
};

struct SyncWords {
    unsigned *counters;   // [(group * 2 + chain) * kSyncStride]
    unsigned *give_up;    // device flag, polled; behind it one word per group: the XCC id its first member ran on (+ 1)
    unsigned *host_flag;  // pinned host word, written once on give-up
    unsigned *fault;      // device word the launch never clears, written on give-up like the two above (a scrap word when the caller has none)
    float *scrap;         // kScrapWords floats nobody reads
    float *exchange;      // backward, split along k: per group 2 chains x 2 buffers x members^2 tiles of 1 KiB
};

// One lane per wavefront talks to the counters.  A wavefront arrives once its own stores are complete; the last of the
// workgroup's four (counted in LDS; the four stay within one unit of each other, so the count never mixes two units)
// bumps the group's counter: one atomic per workgroup and unit on that cache line.
template <bool AGENT>
__device__ __forceinline__ void wave_arrive(unsigned *counter, unsigned *lds_count)
{
    if ((threadIdx.x & 63) == 0) {
        // as assembly: in front of an LDS atomic the compiler drains every load still on its way into LDS (it cannot tell that
        // they go elsewhere), which would stall a unit that has just requested its next tiles
        unsigned before;
        const unsigned at = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned *)lds_count, one = 1u;
        asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)" : "=v"(before) : "v"(at), "v"(one) : "memory");
        if ((before & 3u) == 3u) {
            if (AGENT) __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
            else __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, MYEA_SCOPE_WORKGROUP);
        }
    }
}

// Waits until the counter reaches `target`.  Returns (to every lane) 1 when it did, 0 when the wait gave up here or
// elsewhere.  One lane polls; the poll is a load that bypasses this compute unit's L1 (many wavefronts read the line, few
// write it: reads do not queue behind one another the way atomics on one address do).  The loop - poll, look at the
// give-up flag, count down, raise the flag when the count runs out - is one block of assembly: written in C++, a loop
// with loads in it makes the compiler's wait-count bookkeeping pessimistic for what follows (it drains all memory
// operations in front of the first MFMA).  Only lane 0 is active in the block, so vcc holds just its compare result.
__device__ __forceinline__ int wave_wait(const SyncWords &w, unsigned *counter, unsigned target, unsigned spin_polls)
{
    int ok = 1;
    if ((threadIdx.x & 63) == 0) {
        unsigned value, polls = spin_polls;
        asm volatile(
            "v_mov_b32 %[ok], 0\n"
            "1:\n\t"
            "global_load_dword %[value], %[counter], off sc1\n\t"
            "s_waitcnt vmcnt(0)\n\t"
            "v_sub_u32 %[value], %[value], %[target]\n\t"
            "v_cmp_le_i32 vcc, 0, %[value]\n\t"
            "s_cbranch_vccnz 2f\n\t"
            "global_load_dword %[value], %[give_up], off sc1\n\t"
            "s_waitcnt vmcnt(0)\n\t"
            "v_cmp_ne_u32 vcc, 0, %[value]\n\t"
            "s_cbranch_vccnz 3f\n\t"
            "s_sleep 2\n\t"
            "s_sub_u32 %[polls], %[polls], 1\n\t"
            "s_cmp_lg_u32 %[polls], 0\n\t"
            "s_cbranch_scc1 1b\n\t"
            "v_mov_b32 %[value], 1\n\t"
            "global_store_dword %[give_up], %[value], off sc1\n\t"
            "global_store_dword %[host_flag], %[value], off sc0 sc1\n\t"
            "global_store_dword %[fault], %[value], off sc1\n\t"
            "s_waitcnt vmcnt(0)\n\t"
            "s_branch 3f\n"
            "2:\n\t"
            "v_mov_b32 %[ok], 1\n"
            "3:\n"
            : [ok] "=&v"(ok), [value] "=&v"(value), [polls] "+s"(polls)
            : [counter] "v"(counter), [give_up] "v"(w.give_up), [host_flag] "v"(w.host_flag), [fault] "v"(w.fault), [target] "v"(target)
            : "vcc", "scc", "memory");
    }
    return __builtin_amdgcn_readfirstlane(ok);
}

__device__ __forceinline__ unsigned xcc_id() { return __builtin_amdgcn_s_getreg(20 | (3 << 11)) & 15u; }   // HW_REG_XCC_ID[3:0]

// workgroup id -> (group, member).  LOCAL: the XCD of ids = x (mod 8) hosts the groups x, x + 8, ...; AGENT: members of a
// group are spread over the XCDs.  Returns false for a workgroup without work.
// f(integral_constant<int, I>{}) for I = FIRST .. LAST - 1, unrolled
template <int FIRST, int LAST, class F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (FIRST < LAST) {
        f(std::integral_constant<int, FIRST>{});
        static_for<FIRST + 1, LAST>(f);
    }
}

template <bool AGENT>
__device__ __forceinline__ bool place(unsigned id, int members, int groups, int &group, int &member)
{
    if (AGENT) { group = (int)(id % (unsigned)groups); member = (int)(id / (unsigned)groups); return member < members; }
    const int xcd = (int)(id & 7), slot = (int)(id >> 3);
    group = (slot / members) * 8 + xcd;
    member = slot % members;
    return group < groups;
}

// LOCAL: every member of the group must sit on the same XCD (which one depends on the hardware queue the launch went
// through): the first member to get here writes its XCC id, the others compare.  A member elsewhere does not share the
// group's L2: it stops everybody.
__device__ __forceinline__ void check_same_xcd(const SyncWords &w, int group)
{
    if (threadIdx.x != 0) return;
    unsigned *word = w.give_up + 1 + group;
    const unsigned mine = xcc_id() + 1u;
    unsigned seen = 0u;
    if (!__hip_atomic_compare_exchange_strong(word, &seen, mine, __ATOMIC_RELAXED, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT) && seen != mine) {
        __hip_atomic_store(w.give_up, 1u, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
        __hip_atomic_store(w.host_flag, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __hip_atomic_store(w.fault, 1u, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
    }
}

}  // namespace

struct ResidentGeometry {
    int T, B, Bmax, C;
    int dirs, row_groups;      // groups = dirs * row_groups; group g: direction g % dirs, examples from (g / dirs) * 2 ROWS
    int members;               // workgroups per group = C / CELLS
    int arrivals;              // arrivals that complete a unit: members (one more under the test switch, so that no unit ever completes)
    unsigned spin_polls;       // polls after which a wait gives up
    int never_early;           // test switch: the look at the other chain's counter during a unit's MFMAs always says "not yet"
};

namespace {

// ---- forward ---------------------------------------------------------------------------------------------------------
// KW = C / 4: k's per wavefront.  Chain 0 holds the group's first ROWS examples, chain 1 the next ROWS.
// Per lane the addresses of its (example, cell) pair(s) and of its tile rows are set up once and then stepped.
using Chain0 = std::integral_constant<int, 0>;
using Chain1 = std::integral_constant<int, 1>;

template <int KW, int CELLS, int RS, bool AGENT>
__global__ __launch_bounds__(kThreads, 1) void lstm_resident_forward_kernel(ResidentGeometry g, LstmResidentDir d0, LstmResidentDir d1, SyncWords w)
{
    constexpr int C = 4 * KW, G = 4 * C;
    constexpr int NB = 4 * CELLS, NCT = NB / 16, ROWS = 16 * RS, NT = KW / 32;
    constexpr int LPT = ROWS / 8;                 // direct loads per tile
    constexpr int PAIRS = ROWS * CELLS / kThreads;
    constexpr int NSTORE = 7 * PAIRS;             // stores of a unit
    constexpr int A1 = NT >= 4 ? NT / 4 : 1;      // tiles whose MFMAs run before the previous unit's arrival is signalled
    constexpr int P1 = NT >= 4 ? (3 * NT) / 4 : NT - 1;   // tile before which the next unit's counter is read
    constexpr int kStride = NB + 8;               // floats per row of a wavefront's partial tile
    constexpr bool HALF = !AGENT && NT == 4 && RS == 1;   // 512 cells: a unit's four tiles are requested in two halves, each two tiles of MFMAs ahead
    constexpr int SLOTS = NT;
    constexpr int kAhead = HALF ? NT / 2 : NT;    // tiles of a unit that the other chain requests for it
    constexpr int kStage = SLOTS * ROWS * 32, kPart = 4 * ROWS * kStride;
    constexpr int kAux = AGENT ? 16 : kLocalAux;
    constexpr bool DB = AGENT;                    // the other chain's tiles are requested during this chain's last MFMAs, into the slots those have left
    constexpr int S1 = (5 * NT) / 8, X1 = (3 * NT) / 4;   // DB: tile behind which the other chain's counter is read / behind which its value is looked at
    static_assert(!DB || (NT >= 8 && X1 > S1 && X1 < NT && X1 % (NT - X1) == 0), "tiles left to spread the requests over");
    static_assert(PAIRS >= 1 && ROWS * CELLS % kThreads == 0, "every lane has the same number of pairs");
    static_assert(NT * LPT + NSTORE < 64, "vmcnt has 6 bits");
    extern __shared__ __attribute__((aligned(16))) float smem[];
    __shared__ unsigned s_arrive[2];   // wavefronts that arrived, per chain
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col16 = lane & 15, quad = lane >> 4;

    int group, member;
    if (!place<AGENT>(blockIdx.x, g.members, g.dirs * g.row_groups, group, member)) return;
    const int dir = group % g.dirs, rg = group / g.dirs;
    const LstmResidentDir &d = dir ? d1 : d0;
    const int c0 = member * CELLS, B = g.B, T = g.T;
    const size_t Bmax = (size_t)g.Bmax;
    unsigned *const counters = w.counters + (size_t)group * 2 * kSyncStride;   // chain c: counters + c * kSyncStride
    const unsigned members = (unsigned)g.arrivals;
    if (!AGENT) check_same_xcd(w, group);
    if (threadIdx.x < 2) s_arrive[threadIdx.x] = 0u;
    __syncthreads();

    float *const stage = smem + wave * kStage;   // this wavefront's tiles of the unit in flight
    float *const parts = smem + 4 * kStage;      // [chain][4 wavefronts][ROWS][kStride]

    // the weight slice: gate column j = ct * 16 + col16 of the workgroup is gate j / CELLS of cell c0 + j % CELLS
    f32x4 breg[NT][2][NCT];
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) {
        const int j = ct * 16 + col16;
        const float *row = d.Wrec + ((size_t)(j / CELLS) * C + c0 + (j % CELLS)) * C + wave * KW;
#pragma unroll
        for (int i = 0; i < NT; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h) breg[i][h][ct] = *reinterpret_cast<const f32x4 *>(row + i * 32 + (h * 4 + quad) * 4);
    }
    const int t_first = d.reverse ? T - 1 : 0;
    const ptrdiff_t t_step = d.reverse ? -1 : 1;
    const ptrdiff_t step_g = t_step * (ptrdiff_t)(Bmax * G), step_c = t_step * (ptrdiff_t)(Bmax * C);
    const ptrdiff_t zone_step = t_step * (ptrdiff_t)d.zone_stride;
    // the lane's pairs: constants shared by the chains; per chain the state carried from step to step and the addresses
    float e_bias[PAIRS][4], e_peep[PAIRS][3];
    float c_prev[2][PAIRS], h_prev[2][PAIRS], e_in[PAIRS][4];
    unsigned keep_c[PAIRS], keep_h[PAIRS];   // 0: a zoned-out cell keeps its previous state / output at this step
    float *p_acts[2][PAIRS], *p_c[2][PAIRS], *p_ca[2][PAIRS], *p_h[2][PAIRS];
    ptrdiff_t lane_step_c[2][PAIRS];   // 0 for a lane whose stores go to the scrap area
    const unsigned char *p_zone_c[PAIRS], *p_zone_h[PAIRS];   // chain 0's step; chain 1 is at the same one or one behind
    const float *p_tile[2][LPT];
#pragma unroll
    for (int q = 0; q < PAIRS; ++q) {
        const int pair = threadIdx.x + q * kThreads, row = pair / CELLS, cell = pair % CELLS, k = c0 + cell;
#pragma unroll
        for (int gate = 0; gate < 4; ++gate) e_bias[q][gate] = d.bias[gate * C + k];
#pragma unroll
        for (int gate = 0; gate < 3; ++gate) e_peep[q][gate] = d.peep[gate * C + k];
        p_zone_c[q] = d.zone_state ? d.zone_state + (size_t)t_first * d.zone_stride + k : nullptr;
        p_zone_h[q] = d.zone_output ? d.zone_output + (size_t)t_first * d.zone_stride + k : nullptr;
#pragma unroll
        for (int ch = 0; ch < 2; ++ch) {
            const int r = (rg * 2 + ch) * ROWS + row;
            const bool valid = r < B;
            const size_t at = (size_t)t_first * Bmax + min(r, B - 1);
            float *scrap = w.scrap + 4096 + (ch * PAIRS + q) * kThreads + threadIdx.x;
            p_acts[ch][q] = d.acts + at * G + k;   // the input sums; a lane without an example reads the batch's last example's
            p_c[ch][q] = valid ? d.c + at * C + k : scrap;
            p_ca[ch][q] = valid ? d.ca + at * C + k : scrap + 1024;
            p_h[ch][q] = valid ? d.h + at * C + k : scrap + 2048;
            lane_step_c[ch][q] = valid ? step_c : 0;
            c_prev[ch][q] = 0.f; h_prev[ch][q] = 0.f;
        }
    }
    // where the gate activations go: over the input sums, or for a lane without an example to the scrap area
    float *p_acts_out[2][PAIRS];
    ptrdiff_t lane_step_out[2][PAIRS];
#pragma unroll
    for (int q = 0; q < PAIRS; ++q)
#pragma unroll
        for (int ch = 0; ch < 2; ++ch) {
            const int pair = threadIdx.x + q * kThreads, r = (rg * 2 + ch) * ROWS + pair / CELLS;
            p_acts_out[ch][q] = r < B ? p_acts[ch][q] : w.scrap + (ch * PAIRS + q) * kThreads + threadIdx.x;
            lane_step_out[ch][q] = r < B ? step_g : 0;
        }
    // rows of h the wavefront stages (clamped to the batch), at the direction's first step
#pragma unroll
    for (int ch = 0; ch < 2; ++ch)
#pragma unroll
        for (int q = 0; q < LPT; ++q) {
            const int r = q * 8 + (lane >> 3), chunk = (lane & 7) ^ ((r >> 1) & 7);
            p_tile[ch][q] = d.h + ((size_t)t_first * Bmax + min((rg * 2 + ch) * ROWS + r, B - 1)) * C + wave * KW + chunk * 4;
        }

    f32x4 acc[RS][NCT];
    unsigned seen = 0;   // the next unit's counter as read during the MFMAs

    auto load_inputs = [&](auto ch) {   // input sums (and zoneout masks) of the step the chain's pointers are at
        constexpr int c = decltype(ch)::value;
#pragma unroll
        for (int q = 0; q < PAIRS; ++q) {
#pragma unroll
            for (int gate = 0; gate < 4; ++gate) e_in[q][gate] = p_acts[c][q][gate * C];
            keep_c[q] = 1u; keep_h[q] = 1u;
        }
        if (d.zone_state) {
#pragma unroll
            for (int q = 0; q < PAIRS; ++q) keep_c[q] = p_zone_c[q][0];
        }
        if (d.zone_output) {
#pragma unroll
            for (int q = 0; q < PAIRS; ++q) keep_h[q] = p_zone_h[q][0];
        }
    };
    // tiles [first, last) of h of the step before the one the chain's pointers are at (p_tile is one step behind);
    // `advance`: these were the step's last tiles
    auto load_tile_range = [&](auto ch, auto first, auto last, auto advance) {
        constexpr int c = decltype(ch)::value;
#pragma unroll
        for (int i = decltype(first)::value; i < decltype(last)::value; ++i)
#pragma unroll
            for (int q = 0; q < LPT; ++q)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(p_tile[c][q] + i * 32),
                                                 (__attribute__((address_space(3))) void *)(stage + (i % SLOTS) * ROWS * 32 + q * 256), 16, 0, kAux);
        if (decltype(advance)::value) {
#pragma unroll
            for (int q = 0; q < LPT; ++q) p_tile[c][q] += step_c;
        }
    };
    auto load_tiles = [&](auto ch) { load_tile_range(ch, std::integral_constant<int, 0>{}, std::integral_constant<int, kAhead>{}, std::integral_constant<bool, !HALF>{}); };
    auto mfma_tiles = [&](auto ch, auto first, auto last) {
#pragma unroll
        for (int i = decltype(first)::value; i < decltype(last)::value; ++i) {
            const float *tile = stage + (i % SLOTS) * ROWS * 32;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                f32x4 fa[RS];
#pragma unroll
                for (int rs = 0; rs < RS; ++rs) fa[rs] = ATile<ROWS, kAux>::chunk(tile, rs * 16 + col16, h * 4 + quad);
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                        for (int rs = 0; rs < RS; ++rs)
                            acc[rs][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[rs][e], breg[i][h][ct][e], acc[rs][ct], 0, 0, 0);
            }
        }
    };
    using I0 = std::integral_constant<int, 0>;
    using IA = std::integral_constant<int, A1>;
    using IP = std::integral_constant<int, (P1 > A1 ? P1 : A1)>;
    using IN = std::integral_constant<int, NT>;

    // The first part of a unit with a recurrent term: its tiles have landed when only the previous unit's stores can be
    // outstanding; after a quarter of the MFMAs those stores are complete too and the previous unit - of the other chain -
    // arrives.  all_landed: nothing may be outstanding (after the first units, whose requests were made in another order).
    auto head = [&](auto ch, auto all_landed) {
        constexpr int c = decltype(ch)::value;
#pragma unroll
        for (int rs = 0; rs < RS; ++rs)
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) acc[rs][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (decltype(all_landed)::value) wait_vm<0>(); else wait_vm<NSTORE>();
        if constexpr (HALF) {   // the unit's second half: the third tile now, the fourth behind the first tile's MFMAs - two tiles of MFMAs ahead each
            __builtin_amdgcn_sched_barrier(0);
            load_tile_range(ch, std::integral_constant<int, 2>{}, std::integral_constant<int, 3>{}, std::false_type{});
            __builtin_amdgcn_sched_barrier(0);
        }
        mfma_tiles(ch, I0{}, IA{});
        __builtin_amdgcn_sched_barrier(0);   // keeps the MFMAs above in front of the wait
        if constexpr (HALF) {   // the stores of the unit before are older than the two requests
            load_tile_range(ch, std::integral_constant<int, 3>{}, IN{}, std::true_type{});
            __builtin_amdgcn_sched_barrier(0);
            wait_vm<2 * LPT>();
        } else {
            wait_vm<0>();
        }
        wave_arrive<AGENT>(counters + (1 - c) * kSyncStride, &s_arrive[1 - c]);
    };
    // The rest of the unit.  FIRST: the chain's first step (no recurrent term, no forget gate, no peephole into the input
    // gate).  wait_for: the other chain's units that must have arrived before its next unit's tiles are requested (0: that
    // unit has no recurrent term, or there is none).  Returns false when a wait gave up.
    auto tail = [&](auto ch, auto first_tag, unsigned wait_for) -> bool {
        constexpr int c = decltype(ch)::value;
        constexpr bool FIRST = decltype(first_tag)::value;
        load_inputs(ch);
        bool requested = false;   // the other chain's tiles are on their way already
        if constexpr (!FIRST && HALF) {
            // A unit's four tiles are requested two at a time (its first two behind the last two MFMA tiles of the unit before, if
            // the chain's counter is complete by then; the third and the fourth in the unit's head, around its first tile's
            // MFMAs), so a wavefront never issues more than two loads in a row - eight in a row, four wavefronts at once, keep
            // the compute unit's address path busy for 512 clocks during which the issuing wavefronts stand still - and every tile
            // has two tiles of MFMAs to arrive (with one, the wait for it cost 500 clocks a tile).  The first wait counts what
            // was issued behind the tile it waits for: the fourth tile, the counter, and the unit's inputs, counted as four loads,
            // the fewest there can be (two more with zoneout masks: it then asks for a little more than it needs).  The second leaves nothing in flight - the inputs too, requested two
            // tiles of MFMAs ago - so that the compiler has no load left to wait for in front of the gate math: it would
            // wait for everything there, the next unit's tiles included.
            constexpr int kIn = 4 * PAIRS;
            using I1 = std::integral_constant<int, 1>;
            using I2 = std::integral_constant<int, 2>;
            using I3 = std::integral_constant<int, 3>;
            using Other = std::integral_constant<int, 1 - c>;
            __builtin_amdgcn_sched_barrier(0);
            mfma_tiles(ch, I1{}, I2{});
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("global_load_dword %0, %1, off sc1" : "=v"(seen) : "v"(counters + (1 - c) * kSyncStride) : "memory");
            __builtin_amdgcn_sched_barrier(0);
            wait_vm<LPT + 1 + kIn>();              // the third tile has landed: behind it came the inputs, the fourth tile, the counter
            mfma_tiles(ch, I2{}, I3{});
            __builtin_amdgcn_sched_barrier(0);
            wait_vm<0>();                          // the fourth, the counter's value, the inputs
            asm volatile("" : "+v"(seen));         // looked at behind the wait, not before
            if (wait_for && !g.never_early && (int)(__builtin_amdgcn_readfirstlane(seen) - wait_for * members) >= 0) {
                load_tile_range(Other{}, I0{}, I1{}, std::false_type{});
                __builtin_amdgcn_sched_barrier(0);
                mfma_tiles(ch, I3{}, IN{});
                __builtin_amdgcn_sched_barrier(0);
                load_tile_range(Other{}, I1{}, I2{}, std::false_type{});
                requested = true;
            } else {
                mfma_tiles(ch, I3{}, IN{});
            }
            __builtin_amdgcn_sched_barrier(0);
        } else if constexpr (!FIRST && DB) {
            // The other chain's counter is read five eighths into the MFMAs, when its step is normally complete, and looked at an
            // eighth later; its tiles are then requested between the last quarter's MFMAs, into the slots whose tiles those
            // MFMAs no longer need (a tile's own slot right behind its MFMAs) - they have those MFMAs and the gate math to
            // arrive, and the requests do not come as one burst (a compute unit's address path takes 16 clocks per 1 KiB load
            // instruction; a wavefront that issues sixteen in a row stands still meanwhile).
            using IS = std::integral_constant<int, S1>;
            using IX = std::integral_constant<int, X1>;
            __builtin_amdgcn_sched_barrier(0);
            mfma_tiles(ch, IA{}, IS{});
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("global_load_dword %0, %1, off sc1" : "=v"(seen) : "v"(counters + (1 - c) * kSyncStride) : "memory");
            mfma_tiles(ch, IS{}, IX{});
            __builtin_amdgcn_sched_barrier(0);
            wait_vm<0>();                          // the unit's inputs (requested long ago) and the counter's value
            asm volatile("" : "+v"(seen));         // looked at behind the wait, not before
            if (wait_for && !g.never_early && (int)(__builtin_amdgcn_readfirstlane(seen) - wait_for * members) >= 0) {
                constexpr int kEach = X1 / (NT - X1);   // free slots filled per tile of MFMAs
                static_for<X1, NT>([&](auto i) {
                    constexpr int I = decltype(i)::value;
                    __builtin_amdgcn_sched_barrier(0);
                    mfma_tiles(ch, i, std::integral_constant<int, I + 1>{});
                    __builtin_amdgcn_sched_barrier(0);
                    load_tile_range(std::integral_constant<int, 1 - c>{}, std::integral_constant<int, (I - X1) * kEach>{},
                                    std::integral_constant<int, (I - X1 + 1) * kEach>{}, std::false_type{});
                    load_tile_range(std::integral_constant<int, 1 - c>{}, i, std::integral_constant<int, I + 1>{}, std::integral_constant<bool, I + 1 == NT>{});
                });
                requested = true;
            } else {
                mfma_tiles(ch, IX{}, IN{});
            }
            __builtin_amdgcn_sched_barrier(0);
        } else if (!FIRST) {
            mfma_tiles(ch, IA{}, IP{});
            if (wait_for) seen = __hip_atomic_load(counters + (1 - c) * kSyncStride, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
            mfma_tiles(ch, IP{}, IN{});
            __builtin_amdgcn_sched_barrier(0);   // the counter's value is looked at after the MFMAs, not right behind its load
        }
        if (wait_for && !requested) {
            const unsigned target = wait_for * members;
            const bool there = !FIRST && !DB && !HALF && (int)(__builtin_amdgcn_readfirstlane(seen) - target) >= 0;
            if (!there && !wave_wait(w, counters + (1 - c) * kSyncStride, target, g.spin_polls)) return false;
            load_tiles(std::integral_constant<int, 1 - c>{});   // every wavefront's reads of this unit's tiles have been issued and waited for by its MFMAs
        }
        float *part = parts + c * kPart;
        if (!FIRST) {
            float *to = part + wave * ROWS * kStride;
#pragma unroll
            for (int rs = 0; rs < RS; ++rs)
#pragma unroll
                for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
                    for (int r = 0; r < 4; ++r) to[(rs * 16 + quad * 4 + r) * kStride + ct * 16 + col16] = acc[rs][ct][r];
            lds_barrier();
        }
#pragma unroll
        for (int q = 0; q < PAIRS; ++q) {
            const int pair = threadIdx.x + q * kThreads, row = pair / CELLS, cell = pair % CELLS;
            float rec[4] = {0.f, 0.f, 0.f, 0.f};
            if (!FIRST) {
#pragma unroll
                for (int gate = 0; gate < 4; ++gate) {
                    float v = 0.f;
#pragma unroll
                    for (int wv = 0; wv < 4; ++wv) v += part[(wv * ROWS + row) * kStride + gate * CELLS + cell];
                    rec[gate] = v;
                }
            }
            const float cp = c_prev[c][q];
            float si = e_in[q][1] + rec[1] + e_bias[q][1];
            float gf = 0.f;
            if (!FIRST) {
                float sf = e_in[q][2] + rec[2] + e_bias[q][2];
                si += cp * e_peep[q][0];
                sf += cp * e_peep[q][1];
                gf = sigmoid_f(sf);
            }
            const float gi = sigmoid_f(si);
            const float z = tanh_f(e_in[q][0] + rec[0] + e_bias[q][0]);
            float cs = FIRST ? z * gi : z * gi + gf * cp;
            cs = keep_c[q] ? cs : cp;   // a zoned-out cell state keeps the previous one (0 on the first step)
            const float a = tanh_f(cs);
            const float so = e_in[q][3] + rec[3] + e_bias[q][3] + cs * e_peep[q][2];
            const float go = sigmoid_f(so);
            float hv = a * go;
            hv = keep_h[q] ? hv : h_prev[c][q];
            c_prev[c][q] = cs; h_prev[c][q] = hv;
            if (AGENT) __hip_atomic_store(p_h[c][q], hv, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
            else *p_h[c][q] = hv;
            float *arow = p_acts_out[c][q];
            arow[0] = z; arow[C] = gi; arow[2 * C] = gf; arow[3 * C] = go;
            *p_c[c][q] = cs; *p_ca[c][q] = a;
            p_h[c][q] += lane_step_c[c][q]; p_c[c][q] += lane_step_c[c][q]; p_ca[c][q] += lane_step_c[c][q];
            p_acts[c][q] += step_g; p_acts_out[c][q] += lane_step_out[c][q];
        }
        if (c == 1) {   // both chains have used this step's masks
#pragma unroll
            for (int q = 0; q < PAIRS; ++q) { if (d.zone_state) p_zone_c[q] += zone_step; if (d.zone_output) p_zone_h[q] += zone_step; }
        }
        return true;
    };
    using First = std::true_type;
    using Later = std::false_type;

    // units in program order: (0,0) (1,0) (0,1) (1,1) ... ; unit (c, s) needs every member's h of unit (c, s - 1)
    if (!tail(Chain0{}, First{}, 0u)) return;
    wait_vm<0>();
    wave_arrive<AGENT>(counters, &s_arrive[0]);          // unit (0, 0)
    if (!tail(Chain1{}, First{}, 1u)) return;            // requests the tiles of unit (0, 1)
    head(Chain0{}, std::true_type{});                    // signals unit (1, 0)
    for (int s = 1; s + 1 < T; ++s) {
        if (!tail(Chain0{}, Later{}, (unsigned)s)) return;          // chain 1 has arrived s times: tiles of unit (1, s)
        head(Chain1{}, std::false_type{});                          // signals unit (0, s)
        if (!tail(Chain1{}, Later{}, (unsigned)s + 1u)) return;     // tiles of unit (0, s + 1)
        head(Chain0{}, std::false_type{});                          // signals unit (1, s)
    }
    if (!tail(Chain0{}, Later{}, (unsigned)(T - 1))) return;
    head(Chain1{}, std::false_type{});
    if (!tail(Chain1{}, Later{}, 0u)) return;
}

// ---- backward --------------------------------------------------------------------------------------------------------
// The seven sums every lane of a backward workgroup has gathered over its examples (lane = 16 * example + cell within a
// wavefront's 64) folded over the workgroup's examples in a fixed order and left at out[(row_group * 7 + v) * C + c0 + cell]:
// what the weight-gradient pass otherwise reads the gate deltas and cell states once more for.
__device__ __forceinline__ void store_column_sums(const double (&sums)[7], float *out, int row_group, int C, int c0)
{
    if (!out) return;
    __shared__ double s_fold[4][7][16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int v = 0; v < 7; ++v) {
        double x = sums[v];
        x += __shfl_xor(x, 16);
        x += __shfl_xor(x, 32);
        if (lane < 16) s_fold[wave][v][lane] = x;
    }
    __syncthreads();
    if (threadIdx.x < 7 * 16) {
        const int v = threadIdx.x >> 4, cell = threadIdx.x & 15;
        out[((size_t)row_group * 7 + v) * C + c0 + cell] = (float)(((s_fold[0][v][cell] + s_fold[1][v][cell]) + s_fold[2][v][cell]) + s_fold[3][v][cell]);
    }
}

// dh[t] += dG[t'] Wrec (t' = the step processed before t in this pass), then the gate deltas of step t.  The workgroup owns
// CELLS = 16 columns of dh; wavefront w contracts over the k range of gate w (k = gate * C + cell of dG[t']) against its
// slice of the transposed packed matrix WrecT [C][4C].  j counts the steps of this pass: the direction's own step is
// s = T - 1 - j.  j = 0 has no recurrent term and no terms from a later step; s = 0 writes no forget-gate delta.
template <int CC, int RS>
__global__ __launch_bounds__(kThreads, 1) void lstm_resident_backward_kernel(ResidentGeometry g, LstmResidentDir d0, LstmResidentDir d1, SyncWords w)
{
    constexpr int C = CC, G = 4 * C, CELLS = 16;
    constexpr int ROWS = 16 * RS, NT = C / 32;    // tiles of 32 k in a gate's range
    constexpr int LPT = ROWS / 8;
    constexpr int PAIRS = ROWS * CELLS / kThreads;
    constexpr int NSTORE = 6 * PAIRS;
    constexpr int A1 = NT / 4, P1 = (3 * NT) / 4;
    constexpr int kStride = 17;
    // WIDE (C = 1024): a unit's gate deltas (16 examples x 4096 k = 256 KiB) do not fit LDS at once.  They pass through two
    // half buffers of NT / 4 tiles per wavefront in four groups: while group g is contracted, group g + 2 lands in the half
    // that group g has just left.  Its 64 members span two XCDs: device-scope stores of the gate deltas, device-scope
    // counter, tile loads served beyond the XCD's L2 (as in the forward loop of this width).
    constexpr bool AGENT = C > 512;               // 64 members: the group spans two XCDs
    constexpr bool WIDE = C >= 512 && RS == 1;    // a unit's tiles pass through half as many LDS slots, requested a quarter of the unit ahead
    constexpr int SLOTS = WIDE ? NT / 2 : NT, NG = NT / 4;   // tiles of LDS per wavefront; tiles per group
    constexpr int kStage = SLOTS * ROWS * 32, kPart = 4 * ROWS * kStride;
    constexpr int kAux = AGENT ? 16 : kLocalAux;
    static_assert(!WIDE || RS == 1, "the wide form has one set of rows per chain");
    static_assert(NT >= 4 && (WIDE ? 3 * NG * LPT + 9 : NT * LPT) + NSTORE < 64, "vmcnt has 6 bits");
    extern __shared__ __attribute__((aligned(16))) float smem[];
    __shared__ unsigned s_arrive[2];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col16 = lane & 15, quad = lane >> 4;

    int group, member;
    if (!place<AGENT>(blockIdx.x, g.members, g.dirs * g.row_groups, group, member)) return;
    const int dir = group % g.dirs, rg = group / g.dirs;
    const LstmResidentDir &d = dir ? d1 : d0;
    const int c0 = member * CELLS, B = g.B, T = g.T;
    const size_t Bmax = (size_t)g.Bmax;
    unsigned *const counters = w.counters + (size_t)group * 2 * kSyncStride;
    const unsigned members = (unsigned)g.arrivals;
    if (!AGENT) check_same_xcd(w, group);
    if (threadIdx.x < 2) s_arrive[threadIdx.x] = 0u;
    __syncthreads();

    float *const stage = smem + wave * kStage;
    float *const parts = smem + 4 * kStage;

    // WrecT rows c0 .. c0 + 15, the k range of gate `wave`
    f32x4 breg[NT][2];
    {
        const float *row = d.WrecT + (size_t)(c0 + col16) * G + (size_t)wave * C;
#pragma unroll
        for (int i = 0; i < NT; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h) breg[i][h] = *reinterpret_cast<const f32x4 *>(row + i * 32 + (h * 4 + quad) * 4);
    }
    // this pass walks the direction's steps from its last to its first: in time, forwards for the reversed direction
    const int t_first = d.reverse ? 0 : T - 1;
    const ptrdiff_t t_step = d.reverse ? 1 : -1;
    const ptrdiff_t step_g = t_step * (ptrdiff_t)(Bmax * G), step_c = t_step * (ptrdiff_t)(Bmax * C);
    float e_peep[PAIRS][3];
    float n_di[2][PAIRS], n_df[2][PAIRS], n_f[2][PAIRS], n_dc[2][PAIRS];   // of the chain's step processed before: delta i, delta f, f, delta c
    float e_act[PAIRS][4], e_ca[PAIRS], e_cp[PAIRS], e_cs[PAIRS], e_dh[PAIRS];
    double sums[7] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0};   // over the lane's examples and steps: dz, di, df, do, di c', df c', do c (c': the state of the step before)
    const float *p_acts[2][PAIRS], *p_ca[2][PAIRS], *p_cp[2][PAIRS], *p_dh_in[2][PAIRS];   // read: the batch's last example for a lane without one
    float *p_dh[2][PAIRS], *p_dG[2][PAIRS], *p_dc[2][PAIRS];                                  // written: the scrap area for such a lane
    ptrdiff_t lane_step_g[2][PAIRS], lane_step_c[2][PAIRS];
    const float *p_tile[2][LPT];
#pragma unroll
    for (int q = 0; q < PAIRS; ++q) {
        const int pair = threadIdx.x + q * kThreads, row = pair >> 4, cell = pair & 15, k = c0 + cell;
#pragma unroll
        for (int gate = 0; gate < 3; ++gate) e_peep[q][gate] = d.peep[gate * C + k];
#pragma unroll
        for (int ch = 0; ch < 2; ++ch) {
            const int r = (rg * 2 + ch) * ROWS + row;
            const bool valid = r < B;
            const size_t at = (size_t)t_first * Bmax + min(r, B - 1);
            float *scrap = w.scrap + (ch * PAIRS + q) * kThreads + threadIdx.x;
            p_acts[ch][q] = d.acts + at * G + k;
            p_ca[ch][q] = d.ca + at * C + k;
            p_cp[ch][q] = d.c + at * C + k + step_c;   // the cell state of the step before t in the direction's order: one step further along this pass
            p_dh_in[ch][q] = d.dh + at * C + k;
            p_dh[ch][q] = valid ? d.dh + at * C + k : scrap + 4096;
            p_dG[ch][q] = valid ? d.dG + at * G + k : scrap;
            p_dc[ch][q] = valid ? d.dc + at * C + k : scrap + 4096 + 1024;
            lane_step_g[ch][q] = valid ? step_g : 0;
            lane_step_c[ch][q] = valid ? step_c : 0;
            n_di[ch][q] = 0.f; n_df[ch][q] = 0.f; n_f[ch][q] = 0.f; n_dc[ch][q] = 0.f;
        }
    }
    // rows of dG the wavefront stages, the k range of its gate, at the pass's first step
#pragma unroll
    for (int ch = 0; ch < 2; ++ch)
#pragma unroll
        for (int q = 0; q < LPT; ++q) {
            const int r = q * 8 + (lane >> 3), chunk = (lane & 7) ^ ((r >> 1) & 7);
            p_tile[ch][q] = d.dG + ((size_t)t_first * Bmax + min((rg * 2 + ch) * ROWS + r, B - 1)) * G + (size_t)wave * C + chunk * 4;
        }

    f32x4 acc[RS][2];
    unsigned seen = 0;

    auto load_operands = [&](auto ch, bool with_cp) {   // of the step the chain's pointers are at; with_cp: not the direction's first step, which has no step before it
        constexpr int c = decltype(ch)::value;
#pragma unroll
        for (int q = 0; q < PAIRS; ++q) {
#pragma unroll
            for (int gate = 0; gate < 4; ++gate) e_act[q][gate] = p_acts[c][q][gate * C];
            e_ca[q] = *p_ca[c][q];
            e_dh[q] = *p_dh_in[c][q];
            e_cp[q] = p_cp[c][q][with_cp ? 0 : -step_c];   // without a step before: any valid address, the value is not used
            e_cs[q] = p_cp[c][q][-step_c];
        }
    };
    // tiles [first, last) of the chain's step into their LDS slots (tile i lives in slot i mod SLOTS); `advance`: these were
    // the step's last tiles, the pointers move on to the next step
    auto load_tile_range = [&](auto ch, auto first, auto last, auto advance) {
        constexpr int c = decltype(ch)::value;
#pragma unroll
        for (int i = decltype(first)::value; i < decltype(last)::value; ++i)
#pragma unroll
            for (int q = 0; q < LPT; ++q)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(p_tile[c][q] + i * 32),
                                                 (__attribute__((address_space(3))) void *)(stage + (i % SLOTS) * ROWS * 32 + q * 256), 16, 0, kAux);
        if (decltype(advance)::value) {
#pragma unroll
            for (int q = 0; q < LPT; ++q) p_tile[c][q] += step_g;
        }
    };
    auto load_tiles = [&](auto ch) {   // dG of the chain's step processed before the one its pointers are at: all of it, or (WIDE) its first group
        load_tile_range(ch, std::integral_constant<int, 0>{}, std::integral_constant<int, WIDE ? NG : SLOTS>{}, std::integral_constant<bool, !WIDE>{});
    };
    // WIDE: one tile at a time, the next tile's operand read from LDS while this one's MFMAs run
    auto read_tile = [&](auto i, f32x4 (&fa)[2]) {
        const float *tile = stage + (decltype(i)::value % SLOTS) * ROWS * 32;
#pragma unroll
        for (int h = 0; h < 2; ++h) fa[h] = ATile<ROWS, kAux>::chunk(tile, col16, h * 4 + quad);
    };
    auto mfma_tile = [&](auto i, const f32x4 (&fa)[2]) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[0][e & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[h][e], breg[decltype(i)::value][h][e], acc[0][e & 1], 0, 0, 0);
    };
    auto mfma_tiles = [&](auto first, auto last) {
#pragma unroll
        for (int i = decltype(first)::value; i < decltype(last)::value; ++i) {
            const float *tile = stage + (i % SLOTS) * ROWS * 32;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                f32x4 fa[RS];
#pragma unroll
                for (int rs = 0; rs < RS; ++rs) fa[rs] = ATile<ROWS, kAux>::chunk(tile, rs * 16 + col16, h * 4 + quad);
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int rs = 0; rs < RS; ++rs)
                        acc[rs][e & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[rs][e], breg[i][h][e], acc[rs][e & 1], 0, 0, 0);
            }
        }
    };
    using I0 = std::integral_constant<int, 0>;
    using IA = std::integral_constant<int, A1>;
    using IP = std::integral_constant<int, P1>;
    using IN = std::integral_constant<int, NT>;

    auto head = [&](auto ch, auto all_landed) {
        constexpr int c = decltype(ch)::value;
#pragma unroll
        for (int rs = 0; rs < RS; ++rs) { acc[rs][0] = f32x4{0.f, 0.f, 0.f, 0.f}; acc[rs][1] = f32x4{0.f, 0.f, 0.f, 0.f}; }
        if (decltype(all_landed)::value) wait_vm<0>(); else wait_vm<NSTORE>();   // the unit's first group has landed
        if constexpr (WIDE) {
            // The loads of a tile are issued one tile at a time between the MFMAs, never as a burst: a compute unit's address path
            // takes 16 clocks per 1 KiB load instruction, and a wavefront that issues sixteen of them in a row stands still for
            // as long as sixty-four MFMAs take.  Here: the second group into the second half, which the other chain has left.
            f32x4 fa[2][2];
            read_tile(I0{}, fa[0]);
            static_for<0, NG>([&](auto i) {
                constexpr int I = decltype(i)::value;
                __builtin_amdgcn_sched_barrier(0);
                if (I + 1 < NG) read_tile(std::integral_constant<int, I + 1>{}, fa[(I + 1) & 1]);
                mfma_tile(i, fa[I & 1]);
                load_tile_range(ch, std::integral_constant<int, I + NG>{}, std::integral_constant<int, I + NG + 1>{}, std::false_type{});
            });
            __builtin_amdgcn_sched_barrier(0);
            wait_vm<NG * LPT>();             // the stores of the unit before are older than the second group's loads
        } else {
            mfma_tiles(I0{}, IA{});
            __builtin_amdgcn_sched_barrier(0);   // keeps the MFMAs above in front of the wait
            wait_vm<0>();
        }
        wave_arrive<AGENT>(counters + (1 - c) * kSyncStride, &s_arrive[1 - c]);
    };
    // FIRST: the pass's first step of the chain (no recurrent term, nothing from a later step); s: the direction's step
    auto tail = [&](auto ch, auto first_tag, int s, unsigned wait_for) -> bool {
        constexpr int c = decltype(ch)::value;
        constexpr bool FIRST = decltype(first_tag)::value;
        // WIDE: every unit must issue the same number of loads, the waits count them - where `s` is a literal zero the compiler
        // would drop the load of the state before it
        if (WIDE) asm volatile("" : "+s"(s));
        load_operands(ch, s > 0);
        if constexpr (!FIRST && WIDE) {
            // tile i's MFMAs, then the loads of the tile that takes a slot no longer read: i + 8 of this unit (two groups ahead
            // of its use minus one), or - the last group - tile i - 24 of the other chain's next unit, if that chain's step is
            // complete by then.  The waits count what was issued behind the tile they wait for (two loads per tile, the eight
            // operands, the counter's value, in program order).
            constexpr int kOps = 8 * PAIRS;
            const unsigned target = wait_for * members;
            f32x4 fa[2][2];
            __builtin_amdgcn_sched_barrier(0);
            wait_vm<(NG - 1) * LPT + kOps>();
            read_tile(IA{}, fa[NG & 1]);
            static_for<NG, 3 * NG>([&](auto i) {
                constexpr int I = decltype(i)::value;
                __builtin_amdgcn_sched_barrier(0);
                wait_vm<(I + 1 < 2 * NG ? (NG - 2) * LPT + kOps : (I <= 2 * NG + 1 ? (NG - 2) * LPT : (NG - 2) * LPT + 1))>();
                read_tile(std::integral_constant<int, I + 1>{}, fa[(I + 1) & 1]);
                mfma_tile(i, fa[I & 1]);
                if (I == 2 * NG + 1)   // the other chain's counter, as assembly: the compiler would wait for ALL loads where the value is used
                    asm volatile("global_load_dword %0, %1, off sc1" : "=v"(seen) : "v"(counters + (1 - c) * kSyncStride) : "memory");
                load_tile_range(ch, std::integral_constant<int, I + NG>{}, std::integral_constant<int, I + NG + 1>{}, std::integral_constant<bool, I + 1 == 3 * NG>{});
            });
            __builtin_amdgcn_sched_barrier(0);
            wait_vm<(NG - 2) * LPT>();       // tile 3 NG + 1 has landed, and the counter's value before it
            asm volatile("" : "+v"(seen));      // the value is looked at behind the wait, not before
            if (wait_for && !g.never_early && (int)(__builtin_amdgcn_readfirstlane(seen) - target) >= 0) {
                static_for<3 * NG, NT>([&](auto i) {
                    constexpr int I = decltype(i)::value;
                    __builtin_amdgcn_sched_barrier(0);
                    if (I > 3 * NG && I + 1 < NT) wait_vm<(NG - 2) * LPT>();
                    if (I + 1 < NT) read_tile(std::integral_constant<int, I + 1>{}, fa[(I + 1) & 1]);
                    mfma_tile(i, fa[I & 1]);
                    load_tile_range(std::integral_constant<int, 1 - c>{}, std::integral_constant<int, I - 3 * NG>{}, std::integral_constant<int, I - 3 * NG + 1>{}, std::false_type{});
                });
                __builtin_amdgcn_sched_barrier(0);
            } else {   // the other chain is late (or has no further unit): this unit's last group first, then the wait, then its tiles in a row
                wait_vm<0>();
                mfma_tiles(IP{}, IN{});
                __builtin_amdgcn_sched_barrier(0);
                if (wait_for) {
                    if (!wave_wait(w, counters + (1 - c) * kSyncStride, target, g.spin_polls)) return false;
                    load_tiles(std::integral_constant<int, 1 - c>{});
                }
            }
        } else if (!FIRST) {
            mfma_tiles(IA{}, IP{});
            if (wait_for) seen = __hip_atomic_load(counters + (1 - c) * kSyncStride, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
            mfma_tiles(IP{}, IN{});
            __builtin_amdgcn_sched_barrier(0);   // the counter's value is looked at after the MFMAs, not right behind its load
        }
        if (wait_for && (FIRST || !WIDE)) {
            const unsigned target = wait_for * members;
            const bool there = !FIRST && (int)(__builtin_amdgcn_readfirstlane(seen) - target) >= 0;
            if (!there && !wave_wait(w, counters + (1 - c) * kSyncStride, target, g.spin_polls)) return false;
            load_tiles(std::integral_constant<int, 1 - c>{});
        }
        float *part = parts + c * kPart;
        if (!FIRST) {
            float *to = part + wave * ROWS * kStride;
#pragma unroll
            for (int rs = 0; rs < RS; ++rs)
#pragma unroll
                for (int r = 0; r < 4; ++r) to[(rs * 16 + quad * 4 + r) * kStride + col16] = acc[rs][0][r] + acc[rs][1][r];
            lds_barrier();
        }
#pragma unroll
        for (int q = 0; q < PAIRS; ++q) {
            const int pair = threadIdx.x + q * kThreads, row = pair >> 4, cell = pair & 15;
            float rec = 0.f;
            if (!FIRST) {
#pragma unroll
                for (int wv = 0; wv < 4; ++wv) rec += part[(wv * ROWS + row) * kStride + cell];
            }
            const float dh = e_dh[q] + rec;
            const float z = e_act[q][0], gi = e_act[q][1], gf = e_act[q][2], go = e_act[q][3];
            const float a = e_ca[q];
            const float ddo = go * (1.f - go) * (dh * a);
            float e = dh * go * (1.f - a * a);
            e += e_peep[q][2] * ddo;
            if (!FIRST) {
                e += e_peep[q][0] * n_di[c][q];
                e += e_peep[q][1] * n_df[c][q];
                e += n_dc[c][q] * n_f[c][q];
            }
            const float dz = e * gi * (1.f - z * z);
            const float di = (e * z) * (gi * (1.f - gi));
            const float df = s > 0 ? (e * e_cp[q]) * (gf * (1.f - gf)) : 0.f;
            n_di[c][q] = di; n_df[c][q] = df; n_f[c][q] = gf; n_dc[c][q] = e;
            if (lane_step_g[c][q] != 0) {   // the lane has an example in this chain
                sums[0] += dz; sums[1] += di; sums[2] += df; sums[3] += ddo;
                sums[4] += s > 0 ? di * e_cp[q] : 0.f; sums[5] += df * e_cp[q]; sums[6] += ddo * e_cs[q];
            }
            float *drow = p_dG[c][q];
            if (AGENT) {   // read by members on another XCD
                __hip_atomic_store(drow, dz, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT); __hip_atomic_store(drow + C, di, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
                __hip_atomic_store(drow + 2 * C, df, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT); __hip_atomic_store(drow + 3 * C, ddo, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
            } else {
                drow[0] = dz; drow[C] = di; drow[2 * C] = df; drow[3 * C] = ddo;
            }
            *p_dh[c][q] = dh; *p_dc[c][q] = e;
            p_acts[c][q] += step_g; p_ca[c][q] += step_c; p_cp[c][q] += step_c; p_dh_in[c][q] += step_c;
            p_dG[c][q] += lane_step_g[c][q]; p_dh[c][q] += lane_step_c[c][q]; p_dc[c][q] += lane_step_c[c][q];
        }
        return true;
    };
    using First = std::true_type;
    using Later = std::false_type;

    // units in program order: (0,0) (1,0) (0,1) (1,1) ... (chain, step j of this pass); the direction's step is T - 1 - j
    if (!tail(Chain0{}, First{}, T - 1, 0u)) return;
    wait_vm<0>();
    wave_arrive<AGENT>(counters, &s_arrive[0]);
    if (!tail(Chain1{}, First{}, T - 1, 1u)) return;
    head(Chain0{}, std::true_type{});
    for (int j = 1; j + 1 < T; ++j) {
        if (!tail(Chain0{}, Later{}, T - 1 - j, (unsigned)j)) return;
        head(Chain1{}, std::false_type{});
        if (!tail(Chain1{}, Later{}, T - 1 - j, (unsigned)j + 1u)) return;
        head(Chain0{}, std::false_type{});
    }
    if (!tail(Chain0{}, Later{}, 0, (unsigned)(T - 1))) return;
    head(Chain1{}, std::false_type{});
    if (!tail(Chain1{}, Later{}, 0, 0u)) return;
    store_column_sums(sums, d.sums, rg, C, c0);
}

// ---- backward, one chain per set of four wavefronts --------------------------------------------------------------------
// The same split along the columns of dh, the same group protocol (LOCAL) and the same arithmetic as the kernel above, with
// the two chains of a member in two SETS of four wavefronts instead of alternating in one instruction stream: eight
// wavefronts, two per SIMD, each set running the plain loop of its own chain - wait for the group, stream the gate deltas of
// the step before through LDS into the MFMAs, exchange the partial tiles within the set, gate deltas, stores, arrive.
// Why: a unit's tail - exchange, gate arithmetic, stores, their drain, the group's counter - has no MFMAs at all, and in one
// instruction stream nothing else runs during it.  With a set per chain one chain's tail and waits run under the other's
// MFMAs.  Both sets keep the member's slice of WrecT in registers (2 x C / 4 registers a lane: C <= 512).
// What made it work (each measured at 512 cells x 256 examples, where the one-stream kernel takes 464 us a pass):
//   - The tile loops take TURNS, in one fixed order (s_turn).  Left alone the two sets fall into step - both contracting at
//     half speed, then both in their tails - and stay there: 1005 us.
//   - One wavefront per set polls the group's counter while the other three watch LDS.  Polls that queue at a busy line hold
//     up everything else their compute units ask of memory (a tile step of 1000 clocks instead of 380, every load
//     instruction a few hundred clocks to issue): 755 -> 438 us (524 -> 418 in the final form).
//   - A short pause before the first poll (below): 414 us.
// The four wavefronts of a set meet through a counter in LDS (s_barrier would tie the two chains together); every wait of
// this kernel is bounded by the same count of polls and ends the wavefront through the give-up path.
template <int CC>
__global__ __launch_bounds__(2 * kThreads, 1) void lstm_resident_backward_sets_kernel(ResidentGeometry g, LstmResidentDir d0, LstmResidentDir d1, SyncWords w)
{
    constexpr int C = CC, G = 4 * C, CELLS = 16, ROWS = 16, NT = C / 32, LPT = ROWS / 8;
    constexpr int SLOTS = NT < 8 ? NT : 8;             // tiles of LDS per wavefront
    constexpr int AHEAD = NT <= 8 ? NT : SLOTS - 2;    // tiles requested ahead of the one being contracted
    constexpr int kStride = 17, kStage = SLOTS * ROWS * 32, kPart = 4 * ROWS * kStride;
    static_assert(NT >= 4 && C <= 512 && 2 * AHEAD + 8 < 64, "weights of both sets in registers; vmcnt has 6 bits");
    extern __shared__ __attribute__((aligned(16))) float smem[];
    __shared__ unsigned s_arrive[2], s_meet[2], s_go[2], s_turn;   // s_turn: how many tile loops the member has finished; loop number n is chain n % 2's
    __shared__ double s_fold[8][7][16];
    const int lane = threadIdx.x & 63, col16 = lane & 15, quad = lane >> 4;
    const int wave8 = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), c = wave8 >> 2, wave = wave8 & 3;   // c: the set's chain
    const int tid = (int)threadIdx.x & (kThreads - 1);

    int group, member;
    if (!place<false>(blockIdx.x, g.members, g.dirs * g.row_groups, group, member)) return;
    const int dir = group % g.dirs, rg = group / g.dirs;
    const LstmResidentDir &d = dir ? d1 : d0;
    const int c0 = member * CELLS, B = g.B, T = g.T;
    const size_t Bmax = (size_t)g.Bmax;
    unsigned *const counter = w.counters + ((size_t)group * 2 + c) * kSyncStride;
    const unsigned members = (unsigned)g.arrivals;
    check_same_xcd(w, group);
    if (threadIdx.x < 2) { s_arrive[threadIdx.x] = 0u; s_meet[threadIdx.x] = 0u; s_go[threadIdx.x] = 0u; }
    if (threadIdx.x == 0) s_turn = 0u;
    __syncthreads();

    float *const stage = smem + wave8 * kStage;
    float *const part = smem + 8 * kStage + c * kPart;

    // WrecT rows c0 .. c0 + 15, the k range of gate `wave`
    f32x4 breg[NT][2];
    {
        const float *row = d.WrecT + (size_t)(c0 + col16) * G + (size_t)wave * C;
#pragma unroll
        for (int i = 0; i < NT; ++i)
#pragma unroll
            for (int h = 0; h < 2; ++h) breg[i][h] = *reinterpret_cast<const f32x4 *>(row + i * 32 + (h * 4 + quad) * 4);
    }
    // Offsets into the [T][Bmax][4C] and [T][Bmax][C] tensors as 32-bit unsigned numbers (the host only picks this kernel when
    // they fit) that step by a wrapped-around amount: a uniform base plus one register per lane instead of a pointer each.
    const int t_first = d.reverse ? 0 : T - 1;
    const unsigned step_g = (unsigned)((d.reverse ? 1 : -1) * (int)(Bmax * G)), step_c = (unsigned)((d.reverse ? 1 : -1) * (int)(Bmax * C));
    // the lane's (example, cell) pair of the set's chain
    const int row = tid >> 4, cell = tid & 15, k = c0 + cell;
    const int r = (rg * 2 + c) * ROWS + row;
    const bool valid = r < B;   // a lane without an example reads the batch's last one and stores nothing
    float e_peep[3];
#pragma unroll
    for (int gate = 0; gate < 3; ++gate) e_peep[gate] = d.peep[gate * C + k];
    const unsigned at = (unsigned)t_first * (unsigned)Bmax + (unsigned)min(r, B - 1);
    unsigned off_g = at * G + k, off_c = at * C + k;
    float n_di = 0.f, n_df = 0.f, n_f = 0.f, n_dc = 0.f;   // of the step processed before: delta i, delta f, f, delta c
    double sums[7] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0};
    // rows of dG the wavefront stages: the k range of its gate, at the step this pass processed before the current one
    unsigned off_tile[LPT];
#pragma unroll
    for (int q = 0; q < LPT; ++q) {
        const int tr = q * 8 + (lane >> 3), chunk = (lane & 7) ^ ((tr >> 1) & 7);
        off_tile[q] = ((unsigned)t_first * (unsigned)Bmax + (unsigned)min((rg * 2 + c) * ROWS + tr, B - 1)) * G + (unsigned)wave * C + chunk * 4;
    }
    auto request_tile = [&](auto i) {
        constexpr int I = decltype(i)::value;
#pragma unroll
        for (int q = 0; q < LPT; ++q)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(d.dG + off_tile[q] + I * 32),
                                             (__attribute__((address_space(3))) void *)(stage + (I % SLOTS) * ROWS * 32 + q * 256), 16, 0, kLocalAux);
    };
    // The set's four wavefronts meet: `target` arrivals in the set's LDS word.  Bounded like every wait here.
    auto meet = [&](unsigned target) -> bool {
        int ok = 1;
        if (lane == 0) {
            const unsigned word = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned *)&s_meet[c], one = 1u;
            const unsigned turn_at = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned *)&s_turn;
            unsigned value, polls = g.spin_polls;
            asm volatile(
                "s_waitcnt lgkmcnt(0)\n\t"
                "ds_add_rtn_u32 %[value], %[word], %[one]\n\t"
                "s_waitcnt lgkmcnt(0)\n\t"
                "v_and_b32 %[value], 3, %[value]\n\t"
                "v_cmp_ne_u32 vcc, 3, %[value]\n\t"
                "s_cbranch_vccnz 1f\n\t"
                "ds_add_u32 %[turn], %[one]\n"      // the set's last wavefront through its tiles hands the matrix units on
                "1:\n\t"
                "ds_read_b32 %[value], %[word]\n\t"
                "s_waitcnt lgkmcnt(0)\n\t"
                "v_sub_u32 %[value], %[value], %[target]\n\t"
                "v_cmp_le_i32 vcc, 0, %[value]\n\t"
                "s_cbranch_vccnz 2f\n\t"
                "s_sleep 1\n\t"
                "s_sub_u32 %[polls], %[polls], 1\n\t"
                "s_cmp_lg_u32 %[polls], 0\n\t"
                "s_cbranch_scc1 1b\n\t"
                "v_mov_b32 %[ok], 0\n"
                "2:\n"
                : [ok] "+v"(ok), [value] "=&v"(value), [polls] "+s"(polls)
                : [word] "v"(word), [one] "v"(one), [target] "v"(target), [turn] "v"(turn_at)
                : "vcc", "scc", "memory");
            if (!ok) {
                __hip_atomic_store(w.give_up, 1u, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
                __hip_atomic_store(w.host_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                __hip_atomic_store(w.fault, 1u, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
            }
        }
        return __builtin_amdgcn_readfirstlane(ok) != 0;
    };

    // The matrix units go to one set at a time, in one fixed order for every member of every group: chain 0's unit, chain 1's,
    // chain 0's next ...  Two sets contracting at once run at half speed each, end together and sit through their tails together -
    // and stay in step; members that took their turns in different orders would hold up both chains of their group.  In turns,
    // a set's exchange, gate arithmetic, stores and waits run under the other's MFMAs.  `number`: which tile loop of the member
    // this is; the set's last wavefront through the tiles counts it as done (in meet()).
    auto take_turn = [&](unsigned number) -> bool {
        int ok = 1;
        if (lane == 0) {
            const unsigned turn_at = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned *)&s_turn;
            unsigned value, polls = g.spin_polls;
            asm volatile(
                "1:\n\t"
                "ds_read_b32 %[value], %[turn]\n\t"
                "s_waitcnt lgkmcnt(0)\n\t"
                "v_cmp_eq_u32 vcc, %[number], %[value]\n\t"
                "s_cbranch_vccnz 2f\n\t"
                "s_sleep 1\n\t"
                "s_sub_u32 %[polls], %[polls], 1\n\t"
                "s_cmp_lg_u32 %[polls], 0\n\t"
                "s_cbranch_scc1 1b\n\t"
                "v_mov_b32 %[ok], 0\n"
                "2:\n"
                : [ok] "+v"(ok), [value] "=&v"(value), [polls] "+s"(polls)
                : [turn] "v"(turn_at), [number] "v"(number)
                : "vcc", "scc", "memory");
            if (!ok) {
                __hip_atomic_store(w.give_up, 1u, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
                __hip_atomic_store(w.host_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                __hip_atomic_store(w.fault, 1u, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
            }
        }
        return __builtin_amdgcn_readfirstlane(ok) != 0;
    };

    // The group's counter has reached `target`: the set's first wavefront asks memory, the other three watch a word in LDS.
    // With all four polling - 128 wavefronts on the line that the group's 32 arrivals are added to - a pass took 524 us instead
    // of 418: the polls queue at the line, and what else their compute units ask of memory queues behind them (a tile step of
    // 1000 clocks instead of 380, a few hundred clocks to issue any load).  Bounded; 0 when the wait gave up here or elsewhere.
    auto group_wait = [&](unsigned target) -> bool {
        int ok = 1;
        if (lane == 0) {
            const unsigned go_at = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned *)&s_go[c];
            unsigned value, polls = g.spin_polls;
            if (wave == 0) {
                asm volatile(
                    "1:\n\t"
                    "global_load_dword %[value], %[counter], off sc1\n\t"
                    "s_waitcnt vmcnt(0)\n\t"
                    "v_sub_u32 %[value], %[value], %[target]\n\t"
                    "v_cmp_le_i32 vcc, 0, %[value]\n\t"
                    "s_cbranch_vccnz 2f\n\t"
                    "global_load_dword %[value], %[give_up], off sc1\n\t"   // somebody else of the launch gave up
                    "s_waitcnt vmcnt(0)\n\t"
                    "v_cmp_ne_u32 vcc, 0, %[value]\n\t"
                    "s_cbranch_vccnz 4f\n\t"
                    "s_sleep 4\n\t"
                    "s_sub_u32 %[polls], %[polls], 1\n\t"
                    "s_cmp_lg_u32 %[polls], 0\n\t"
                    "s_cbranch_scc1 1b\n"
                    "4:\n\t"
                    "v_mov_b32 %[ok], 0\n\t"
                    "s_branch 3f\n"
                    "2:\n\t"
                    "ds_write_b32 %[go], %[target]\n"
                    "3:\n"
                    : [ok] "+v"(ok), [value] "=&v"(value), [polls] "+s"(polls)
                    : [counter] "v"(counter), [target] "v"(target), [go] "v"(go_at), [give_up] "v"(w.give_up)
                    : "vcc", "scc", "memory");
            } else {
                asm volatile(
                    "1:\n\t"
                    "ds_read_b32 %[value], %[go]\n\t"
                    "s_waitcnt lgkmcnt(0)\n\t"
                    "v_sub_u32 %[value], %[value], %[target]\n\t"
                    "v_cmp_le_i32 vcc, 0, %[value]\n\t"
                    "s_cbranch_vccnz 2f\n\t"
                    "s_sleep 2\n\t"
                    "s_sub_u32 %[polls], %[polls], 1\n\t"
                    "s_cmp_lg_u32 %[polls], 0\n\t"
                    "s_cbranch_scc1 1b\n\t"
                    "v_mov_b32 %[ok], 0\n"
                    "2:\n"
                    : [ok] "+v"(ok), [value] "=&v"(value), [polls] "+s"(polls)
                    : [target] "v"(target), [go] "v"(go_at)
                    : "vcc", "scc", "memory");
            }
            if (!ok) {
                __hip_atomic_store(w.give_up, 1u, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
                __hip_atomic_store(w.host_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                __hip_atomic_store(w.fault, 1u, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
            }
        }
        return __builtin_amdgcn_readfirstlane(ok) != 0;
    };

    // the operands of the unit at hand: asked for inside the unit's tile loop, behind its last tile request (the pass's first
    // unit, which has no tiles, asks for them up front)
    float e_act[4], e_ca, e_dh, e_cp, e_cs;
    auto load_operands = [&](int s) {   // s: the direction's step the offsets stand at
#pragma unroll
        for (int gate = 0; gate < 4; ++gate) e_act[gate] = d.acts[off_g + gate * C];
        e_ca = d.ca[off_c]; e_dh = d.dh[off_c];
        e_cp = d.c[s > 0 ? off_c + step_c : off_c];   // the cell state of the step before in the direction's order (without one: any valid address, the value is not used)
        e_cs = d.c[off_c];
    };
    load_operands(T - 1);
    bool alive = true;
    for (int j = 0; j < T && alive; ++j) {
        const int s = T - 1 - j;   // the direction's step
        float rec = 0.f;
        if (j > 0) {
            // every member's gate deltas of the step before are in memory
            // A pause of about 2 k clocks in front of the first look at the counter: the group is never complete earlier, and a set
            // that starts to poll right behind its arrival slows the other set's tiles and stores by more than the pause costs
            // (measured at 512 cells x 256 examples: 414 us a pass with it, 720 without; 16, 48 and 80 x 64 clocks: 420, 417, 457)
            __builtin_amdgcn_s_sleep(32);
            if (!group_wait((unsigned)j * members)) { alive = false; break; }
            static_for<0, AHEAD>([&](auto i) { request_tile(i); });   // on their way while the set waits for its turn
            if constexpr (AHEAD == NT) {   // every tile has been asked for: the operands right behind them
                __builtin_amdgcn_sched_barrier(0);
                load_operands(s);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (!take_turn(2u * (unsigned)(j - 1) + (unsigned)c)) { alive = false; break; }
            f32x4 acc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
            static_for<0, NT>([&](auto i) {
                constexpr int I = decltype(i)::value;
                // loads requested behind tile I's: the tiles after it and, once the last tile has been asked for, this unit's own
                // eight operands (the unit before could not ask for them without standing between its arrival and this wait)
                constexpr int kBehind = (I + AHEAD < NT ? AHEAD - 1 : NT - 1 - I) * LPT + (I + AHEAD >= NT ? 8 : 0);
                __builtin_amdgcn_sched_barrier(0);
                wait_vm<kBehind>();
                const float *tile = stage + (I % SLOTS) * ROWS * 32;
                f32x4 fa[2];
#pragma unroll
                for (int h = 0; h < 2; ++h) fa[h] = ATile<ROWS, kLocalAux>::chunk(tile, col16, h * 4 + quad);
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[e & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[h][e], breg[I][h][e], acc[e & 1], 0, 0, 0);
                asm volatile("" : "+v"(acc[0]), "+v"(acc[1]));   // keeps the tile's MFMAs here: without a side effect of their own they would all sink behind the last tile
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (I + AHEAD < NT) request_tile(std::integral_constant<int, I + AHEAD>{});
                if constexpr (I + AHEAD + 1 == NT) {
                    load_operands(s);
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = 0; q < LPT; ++q) off_tile[q] += step_g;
            float *to = part + wave * ROWS * kStride;
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) to[(quad * 4 + rr) * kStride + col16] = acc[0][rr] + acc[1][rr];
            if (!meet(4u * (unsigned)j)) { alive = false; break; }
#pragma unroll
            for (int wv = 0; wv < 4; ++wv) rec += part[(wv * ROWS + row) * kStride + cell];
        }
        const float dh = e_dh + rec;
        const float z = e_act[0], gi = e_act[1], gf = e_act[2], go = e_act[3];
        const float a = e_ca;
        const float ddo = go * (1.f - go) * (dh * a);
        float e = dh * go * (1.f - a * a);
        e += e_peep[2] * ddo;
        if (j > 0) {
            e += e_peep[0] * n_di;
            e += e_peep[1] * n_df;
            e += n_dc * n_f;
        }
        const float dz = e * gi * (1.f - z * z);
        const float di = (e * z) * (gi * (1.f - gi));
        const float df = s > 0 ? (e * e_cp) * (gf * (1.f - gf)) : 0.f;
        n_di = di; n_df = df; n_f = gf; n_dc = e;
        if (valid) {
            sums[0] += dz; sums[1] += di; sums[2] += df; sums[3] += ddo;
            sums[4] += s > 0 ? di * e_cp : 0.f; sums[5] += df * e_cp; sums[6] += ddo * e_cs;
        }
        if (valid) {
            float *drow = d.dG + off_g;
            drow[0] = dz; drow[C] = di; drow[2 * C] = df; drow[3 * C] = ddo;
            d.dh[off_c] = dh; d.dc[off_c] = e;
        }
        off_g += step_g; off_c += step_c;
        if (j + 1 < T) {
            wait_vm<0>();
            wave_arrive<false>(counter, &s_arrive[c]);
        }
    }
    // the seven sums over the member's examples of both chains, in a fixed order; every wavefront takes part, also one
    // that gave up (its sums are not used: the launch is reported as failed)
    if (d.sums) {
#pragma unroll
        for (int v = 0; v < 7; ++v) {
            double x = sums[v];
            x += __shfl_xor(x, 16);
            x += __shfl_xor(x, 32);
            if (lane < 16) s_fold[wave8][v][lane] = x;
        }
    }
    __syncthreads();
    if (d.sums && threadIdx.x < 7 * 16) {
        const int v = threadIdx.x >> 4, cl = threadIdx.x & 15;
        double x = s_fold[0][v][cl];
#pragma unroll
        for (int wv = 1; wv < 8; ++wv) x += s_fold[wv][v][cl];
        d.sums[((size_t)rg * 7 + v) * C + c0 + cl] = (float)x;
    }
}

// ---- backward, the contraction split along k ------------------------------------------------------------------------
// dh[t] += dG[t'] Wrec with every member contracting over ITS OWN 64 k's: the gate deltas of its 16 cells, which it has
// just computed and keeps in LDS - no member reads another's gate deltas.  What it owes the others is its share of every
// column of dh: per unit a [16 examples][C] slab of partial sums, left in an exchange buffer as 1 KiB tiles
// [consumer][producer][16 examples][16 columns]; a member's recurrent term is the sum of the `members` tiles addressed to
// it, taken in a fixed order (repeatable).  Per unit and workgroup that is members KiB read and C / 16 KiB written
// (C = 512: 32 + 32 KiB, register to register) against the 128 KiB of gate deltas the form above brings into LDS, whose
// load instructions - bound by the compute unit's address path, hidden behind nothing - are a third of its time.
// The slice of Wrec a member keeps is [its 64 gate rows][C]: 16 C / 64 registers per lane.
//
// A unit (chain c, step j of the pass): sum the tiles of (c, j) [requested during the other chain's unit] -> gate deltas
// of step j -> own k's to LDS -> MFMAs for step j + 1 (the transposed product: an accumulator holds four consecutive
// columns of one example, one 16-byte store per lane and tile) -> tiles out.  The other chain's tiles are requested
// three quarters into the MFMAs, when its counter is normally complete; a chain's arrival is signalled behind the NEXT
// unit's gate stores, by which time its tile stores have long been acknowledged.  The tiles of a chain alternate between
// two buffers: a member overwrites a tile two steps later, which it can only reach after every member has arrived for
// the step in between, that is after every member has summed the tiles of the step before that.
// Tiles travel through buffer instructions (the compiler keeps count of them, unlike of inline assembly): loads with sc1
// (served beyond this compute unit's L1), plain stores; a group shares one XCD's L2, as in the form above.
constexpr unsigned kBufferWord3 = 0x00020000u;   // raw buffer of dwords
constexpr int kAuxSc1 = 16;

template <int CC>
__global__ __launch_bounds__(kThreads, 1) void lstm_resident_backward_ksplit_kernel(ResidentGeometry g, LstmResidentDir d0, LstmResidentDir d1, SyncWords w)
{
    constexpr int C = CC, G = 4 * C, CELLS = 16, ROWS = 16;
    constexpr int NQ = C / 4;               // columns of dh per wavefront
    constexpr int NCT = NQ / 16;            // tiles of 16 columns per wavefront = consumers it writes to
    constexpr int MEMBERS = C / CELLS;
    constexpr int NIN = MEMBERS / 4;        // producers whose tiles a wavefront sums
    constexpr int NSTORE = 6;               // stores of a unit's gate math, every lane the same (scrap for lanes without an example)
    constexpr int kRow = 68;                // floats per example of the own gate deltas in LDS: [k & 3][k >> 2], padded
    constexpr int kRead = 7, kCheck = 11;   // k steps (of 16) at which the other chain's counter is read and looked at
    constexpr unsigned kTileBytes = ROWS * CELLS * sizeof(float);
    constexpr unsigned kParityBytes = (unsigned)MEMBERS * MEMBERS * kTileBytes;   // one chain's tiles of one step
    static_assert(NCT >= 1 && NIN == NCT, "16 cells per member");
    __shared__ __attribute__((aligned(16))) float s_own[2][ROWS * kRow];      // per chain: its gate deltas of this member's cells
    __shared__ __attribute__((aligned(16))) float s_sum[2][4][ROWS][CELLS];   // per chain and wavefront: the sum of its producers' tiles
    __shared__ unsigned s_arrive[2];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col16 = lane & 15, quad = lane >> 4;

    int group, member;
    if (!place<false>(blockIdx.x, g.members, g.dirs * g.row_groups, group, member)) return;
    const int dir = group % g.dirs, rg = group / g.dirs;
    const LstmResidentDir &d = dir ? d1 : d0;
    const int c0 = member * CELLS, B = g.B, T = g.T;
    const size_t Bmax = (size_t)g.Bmax;
    unsigned *const counters = w.counters + (size_t)group * 2 * kSyncStride;
    const unsigned arrivals = (unsigned)g.arrivals;
    check_same_xcd(w, group);
    if (threadIdx.x < 2) s_arrive[threadIdx.x] = 0u;
    __syncthreads();
    __builtin_amdgcn_s_setprio(3);   // ahead of the wavefronts of a contraction that shares the compute unit: the loop is the critical path

    // the weights of the member's 64 k's (k = gate * 16 + cell: row gate * C + c0 + cell of Wrec [4C][C]) against the
    // wavefront's columns, as the A operand of the transposed product: lane (col16, quad) holds Wrec[k = 4 ks + quad][16 ct + col16]
    float breg[16][NCT];
#pragma unroll
    for (int ks = 0; ks < 16; ++ks) {
        const int k = ks * 4 + quad;
        const float *wrow = d.Wrec + ((size_t)(k >> 4) * C + c0 + (k & 15)) * C + wave * NQ + col16;
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) breg[ks][ct] = wrow[ct * 16];
    }
    // this pass walks the direction's steps from its last to its first: in time, forwards for the reversed direction
    const int t_first = d.reverse ? 0 : T - 1;
    const ptrdiff_t t_step = d.reverse ? 1 : -1;
    const ptrdiff_t step_g = t_step * (ptrdiff_t)(Bmax * G), step_c = t_step * (ptrdiff_t)(Bmax * C);
    const int row = threadIdx.x >> 4, cell = threadIdx.x & 15, kcell = c0 + cell;   // the lane's (example, cell) pair
    float e_peep[3];
#pragma unroll
    for (int gate = 0; gate < 3; ++gate) e_peep[gate] = d.peep[gate * C + kcell];
    float n_di[2], n_df[2], n_f[2], n_dc[2];   // of the chain's step processed before: delta i, delta f, f, delta c
    float e_act[4], e_ca, e_cp, e_cs, e_dh;
    double sums[7] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0};   // over the lane's examples and steps: dz, di, df, do, di c', df c', do c (c': the state of the step before)
    const float *p_acts[2], *p_ca[2], *p_cp[2], *p_dh_in[2];   // read: the batch's last example for a lane without one
    float *p_dh[2], *p_dG[2], *p_dc[2];                          // written: the scrap area for such a lane
    ptrdiff_t lane_step_g[2], lane_step_c[2];
#pragma unroll
    for (int ch = 0; ch < 2; ++ch) {
        const int r = (rg * 2 + ch) * ROWS + row;
        const bool valid = r < B;
        const size_t at = (size_t)t_first * Bmax + min(r, B - 1);
        float *scrap = w.scrap + ch * kThreads + threadIdx.x;
        p_acts[ch] = d.acts + at * G + kcell;
        p_ca[ch] = d.ca + at * C + kcell;
        p_cp[ch] = d.c + at * C + kcell + step_c;   // the cell state of the step before t in the direction's order: one step further along this pass
        p_dh_in[ch] = d.dh + at * C + kcell;
        p_dh[ch] = valid ? d.dh + at * C + kcell : scrap + 4096;
        p_dG[ch] = valid ? d.dG + at * G + kcell : scrap;
        p_dc[ch] = valid ? d.dc + at * C + kcell : scrap + 4096 + 1024;
        lane_step_g[ch] = valid ? step_g : 0;
        lane_step_c[ch] = valid ? step_c : 0;
        n_di[ch] = 0.f; n_df[ch] = 0.f; n_f[ch] = 0.f; n_dc[ch] = 0.f;
    }
    // the group's part of the exchange buffer: [chain][buffer][consumer][producer][16 examples][16 columns]
    const __amdgpu_buffer_rsrc_t exchange =
        __builtin_amdgcn_make_buffer_rsrc(w.exchange + (size_t)group * (4 * (size_t)kParityBytes / sizeof(float)), 0, (int)(4 * kParityBytes), (int)kBufferWord3);
    // byte offsets within one chain's buffer: the tiles addressed to this member from the wavefront's producers, and this
    // member's tiles to the wavefront's consumers
    const unsigned in_lane = ((unsigned)member * MEMBERS + (unsigned)wave * NIN) * kTileBytes + (unsigned)lane * 16u;
    const unsigned out_lane = ((unsigned)(wave * NCT) * MEMBERS + (unsigned)member) * kTileBytes + (unsigned)(col16 * CELLS + quad * 4) * 4u;

    u32x4 tiles[NIN];
    unsigned seen = 0;

    auto load_operands = [&](auto ch, bool with_cp) {   // of the step the chain's pointers are at; with_cp: not the direction's first step, which has no step before it
        constexpr int c = decltype(ch)::value;
#pragma unroll
        for (int gate = 0; gate < 4; ++gate) e_act[gate] = p_acts[c][gate * C];
        e_ca = *p_ca[c];
        e_dh = *p_dh_in[c];
        e_cp = *(with_cp ? p_cp[c] : p_ca[c]);   // no step before the direction's first: any finite value, the forget gate's delta is zero there
        e_cs = p_cp[c][-step_c];
    };
    auto load_tiles = [&](auto ch, int buffer) {
        constexpr int c = decltype(ch)::value;
        const unsigned from = (unsigned)(c * 2 + buffer) * kParityBytes + in_lane;
#pragma unroll
        for (int i = 0; i < NIN; ++i) tiles[i] = __builtin_amdgcn_raw_buffer_load_b128(exchange, (int)(from + (unsigned)i * kTileBytes), 0, kAuxSc1);
    };

    // One unit: step j of the pass for chain c (s: the direction's step).  FIRST: j = 0, no recurrent term and nothing from a
    // later step.  LAST: no step j + 1 follows.  other_target: arrivals of the other chain that complete the tiles of ITS next
    // unit (unused when it has none, or that one is a first step); other_with_cp: that unit is not at the direction's first
    // step.  Returns false when a wait gave up.  Which loads a unit issues depends on its compile-time kind only: a load under
    // a run-time condition would have the compiler wait for it where the two paths meet.
    auto unit = [&](auto ch, auto first_tag, auto last_tag, int j, int s, unsigned other_target, bool other_with_cp) -> bool {
        constexpr int c = decltype(ch)::value;
        constexpr bool FIRST = decltype(first_tag)::value, LAST = decltype(last_tag)::value;
        constexpr bool REQUEST = !(FIRST && c == 0) && !(LAST && c == 1);   // the other chain's next unit exists and sums tiles
        using Other = std::integral_constant<int, 1 - c>;
        const int other_buffer = (j + c) & 1;   // the other chain's next unit is step j (c == 0) or j + 1 (c == 1)
        float rec = 0.f;
        if (!FIRST) {
            f32x4 sum = __builtin_bit_cast(f32x4, tiles[0]);
#pragma unroll
            for (int i = 1; i < NIN; ++i) sum += __builtin_bit_cast(f32x4, tiles[i]);
            *reinterpret_cast<f32x4 *>(&s_sum[c][wave][lane >> 2][(lane & 3) * 4]) = sum;
            lds_barrier();
#pragma unroll
            for (int wv = 0; wv < 4; ++wv) rec += s_sum[c][wv][row][cell];
        }
        const float dh = e_dh + rec;
        const float z = e_act[0], gi = e_act[1], gf = e_act[2], go = e_act[3];
        const float a = e_ca;
        const float ddo = go * (1.f - go) * (dh * a);
        float e = dh * go * (1.f - a * a);
        e += e_peep[2] * ddo;
        if (!FIRST) {
            e += e_peep[0] * n_di[c];
            e += e_peep[1] * n_df[c];
            e += n_dc[c] * n_f[c];
        }
        const float dz = e * gi * (1.f - z * z);
        const float di = (e * z) * (gi * (1.f - gi));
        const float df = s > 0 ? (e * e_cp) * (gf * (1.f - gf)) : 0.f;
        n_di[c] = di; n_df[c] = df; n_f[c] = gf; n_dc[c] = e;
        if (lane_step_g[c] != 0) {   // the lane has an example in this chain
            sums[0] += dz; sums[1] += di; sums[2] += df; sums[3] += ddo;
            sums[4] += s > 0 ? di * e_cp : 0.f; sums[5] += df * e_cp; sums[6] += ddo * e_cs;
        }
        float *drow = p_dG[c];
        drow[0] = dz; drow[C] = di; drow[2 * C] = df; drow[3 * C] = ddo;
        *p_dh[c] = dh; *p_dc[c] = e;
        p_acts[c] += step_g; p_ca[c] += step_c; p_cp[c] += step_c; p_dh_in[c] += step_c;
        p_dG[c] += lane_step_g[c]; p_dh[c] += lane_step_c[c]; p_dc[c] += lane_step_c[c];
        if (!(FIRST && c == 0)) {
            // the tiles the other chain stored at the end of its unit are older than these six stores: they are complete
            // once at most six operations are outstanding, and with them the other chain has arrived
            __builtin_amdgcn_sched_barrier(0);
            wait_vm<NSTORE>();
            wave_arrive<false>(counters + (1 - c) * kSyncStride, &s_arrive[1 - c]);
        }
        if (LAST) {
            // the pass's last step: no MFMAs to hide the other chain's requests behind
            if (REQUEST) {
                load_operands(Other{}, other_with_cp);
                if (!wave_wait(w, counters + (1 - c) * kSyncStride, other_target, g.spin_polls)) return false;
                load_tiles(Other{}, other_buffer);
            }
            return true;
        }
        // own k's for the MFMAs: k = gate * 16 + cell sits at [example][(k & 3) * 16 + (k >> 2)]
        {
            float *own = s_own[c] + row * kRow + (cell & 3) * 16 + (cell >> 2);
            own[0] = dz; own[4] = di; own[8] = df; own[12] = ddo;
        }
        lds_barrier();
        // the next unit in program order is the other chain's: its operands now, its tiles when its counter is complete
        load_operands(Other{}, other_with_cp);
        f32x4 bf[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) bf[q] = *reinterpret_cast<const f32x4 *>(s_own[c] + col16 * kRow + quad * 16 + q * 4);
        f32x4 acc[NCT];
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) acc[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < 16; ++ks) {
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) acc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(breg[ks][ct], bf[ks >> 2][ks & 3], acc[ct], 0, 0, 0);
            if (ks == kRead && REQUEST) seen = __hip_atomic_load(counters + (1 - c) * kSyncStride, __ATOMIC_RELAXED, MYEA_SCOPE_AGENT);
            if (ks == kCheck && REQUEST) {
                __builtin_amdgcn_sched_barrier(0);   // the counter's value is looked at here, not right behind its load
                if ((int)(__builtin_amdgcn_readfirstlane(seen) - other_target) < 0 && !wave_wait(w, counters + (1 - c) * kSyncStride, other_target, g.spin_polls)) return false;
                load_tiles(Other{}, other_buffer);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // tiles out: accumulator ct holds, for example col16, the columns 16 ct + 4 quad .. + 3 of the wavefront's range,
        // which belong to consumer wave * NCT + ct
        const unsigned to = (unsigned)(c * 2 + ((j + 1) & 1)) * kParityBytes + out_lane;
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[ct]), exchange, (int)(to + (unsigned)ct * MEMBERS * kTileBytes), 0, 0);
        return true;
    };
    using First = std::true_type;
    using Later = std::false_type;

    // units in program order: (0,0) (1,0) (0,1) (1,1) ...; unit (c, j), j >= 1, sums the tiles every member stored at the end
    // of unit (c, j - 1).  Chain 1's arrivals are signalled in chain 0's units and the other way round: before unit (0, j)'s
    // MFMAs chain 1 has arrived j times, before unit (1, j)'s chain 0 has arrived j + 1 times.
    load_operands(Chain0{}, true);
    if (!unit(Chain0{}, First{}, Later{}, 0, T - 1, 0u, true)) return;
    if (!unit(Chain1{}, First{}, Later{}, 0, T - 1, arrivals, T > 2)) return;
    for (int j = 1; j + 1 < T; ++j) {
        if (!unit(Chain0{}, Later{}, Later{}, j, T - 1 - j, (unsigned)j * arrivals, true)) return;
        if (!unit(Chain1{}, Later{}, Later{}, j, T - 1 - j, (unsigned)(j + 1) * arrivals, T - 2 - j > 0)) return;
    }
    if (!unit(Chain0{}, Later{}, First{}, T - 1, 0, (unsigned)(T - 1) * arrivals, false)) return;
    if (!unit(Chain1{}, Later{}, First{}, T - 1, 0, 0u, false)) return;
    store_column_sums(sums, d.sums, rg, C, c0);
}

__global__ void resident_probe_kernel(unsigned *table)
{
    if (threadIdx.x == 0) table[blockIdx.x] = xcc_id();
}

__global__ void resident_clear_kernel(unsigned *words, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) words[i] = 0u;
}

// ---- host: what the device offers ---------------------------------------------------------------------------------------
struct ResidentDevice {
    bool probed = false;
    bool usable = false;           // 8 XCDs, workgroup ids equal mod 8 share one
    int cus = 0;
};
std::mutex g_resident_mutex;
ResidentDevice g_resident_device[64];

constexpr size_t kMaxLds = 160 * 1024;   // LDS of a compute unit

// One probe launch per device and process: a grid of one workgroup per compute unit (made so by its LDS size) records the
// XCC id every workgroup ran on.  LOCAL groups are only used when the ids of one residue class mod 8 all ran on one XCD and
// the eight classes on eight different ones (which class lands on which XCD varies with the hardware queue).
int probe_device(ResidentDevice **out)
{
    int dev = -1;
    MYEA_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) { set_last_error("resident LSTM: device ordinal %d out of range", dev); return MYEA_E_DEVICE; }
    std::lock_guard<std::mutex> lock(g_resident_mutex);
    ResidentDevice &r = g_resident_device[dev];
    *out = &r;
    if (r.probed) return MYEA_OK;
    hipDeviceProp_t prop;
    MYEA_HIP_TRY(hipGetDeviceProperties(&prop, dev));
    r.cus = prop.multiProcessorCount;
    r.probed = true;
    if (r.cus < 8 || r.cus % 8 != 0 || r.cus > 1024 || prop.sharedMemPerBlock < kMaxLds) return MYEA_OK;
    unsigned *table = nullptr;
    MYEA_HIP_TRY(hipMalloc(&table, (size_t)r.cus * sizeof(unsigned)));
    std::vector<unsigned> host((size_t)r.cus);
    const size_t lds = 96 * 1024;   // more than half of a compute unit's LDS: one workgroup per compute unit
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(resident_probe_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(resident_probe_kernel, dim3((unsigned)r.cus), dim3(64), lds, 0, table);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpy(host.data(), table, host.size() * sizeof(unsigned), hipMemcpyDeviceToHost);
    (void)hipFree(table);
    if (e != hipSuccess) return hip_fail(e, "resident LSTM probe");
    bool ok = true;
    for (int i = 0; i < r.cus && ok; ++i) ok = host[i] == host[i & 7] && host[i] < 16;
    for (int a = 0; a < 8 && ok; ++a)
        for (int b = a + 1; b < 8 && ok; ++b) ok = host[a] != host[b];
    r.usable = ok;
    return MYEA_OK;
}

}  // namespace

bool device_groups_share_xcd()
{
    ResidentDevice *dev = nullptr;
    return probe_device(&dev) == MYEA_OK && dev && dev->usable;
}

namespace {

// MYEA_LSTM_RESIDENT=0 keeps every layer on one launch per time step
bool resident_disabled()
{
    const char *e = std::getenv("MYEA_LSTM_RESIDENT");
    return e && e[0] == '0';
}

// A wait gives up after this many polls of its counter (a poll is a load served by L2 or memory plus a short sleep: about a
// microsecond); MYEA_LSTM_RESIDENT_SPIN_POLLS overrides the default of 200 000 (a fifth of a second).
unsigned spin_polls()
{
    const char *e = std::getenv("MYEA_LSTM_RESIDENT_SPIN_POLLS");
    if (e && *e) { const unsigned long long v = std::strtoull(e, nullptr, 10); return v < 1 ? 1u : (v > 0x7fffffffull ? 0x7fffffffu : (unsigned)v); }
    return 200000u;
}

// Which resident form the backward loop takes.  Measured on this device (T = 64, microseconds per launch, split along k
// against split along the columns of dh): with every compute unit busy the column form wins (512 cells x 256 examples: 594
// against 523; 256 x 512: 405 against 392), with half of them or fewer the k form does (512 x 64: 408 against 450;
// 256 x 128: 236 against 267; 128 x 256: 179 against 190) - its exchange is lighter, but what bounds both under full load
// is the tail latency of the operands streamed from memory, which stalls a group at one more barrier per step in the k form.
// The k form needs 17 KB of LDS where the column form needs 140: it is also the one a contraction's workgroups fit beside
// on a compute unit, so a caller that runs weight contractions next to the loop asks for it (plan.ksplit_available).
// MYEA_LSTM_BACKWARD_KSPLIT=0 / 1 forces the column form / the k form wherever it exists.
int ksplit_choice()   // -1: by occupancy, 0: never, 1: always
{
    const char *e = std::getenv("MYEA_LSTM_BACKWARD_KSPLIT");
    return !e || !*e ? -1 : e[0] == '0' ? 0 : 1;
}

// MYEA_LSTM_RESIDENT_TEST_ABSENT_MEMBER=1 makes every group expect one member more than it has: its first wait runs out of
// polls, the kernel ends through its give-up path and the host reports it.  For tests of that path; every wavefront still
// exits normally.
bool absent_member_for_test()
{
    const char *e = std::getenv("MYEA_LSTM_RESIDENT_TEST_ABSENT_MEMBER");
    return e && e[0] == '1';
}

// MYEA_LSTM_RESIDENT_TEST_NEVER_EARLY=1: a unit never finds the other chain's counter complete while its own MFMAs run, so
// the next unit's first tiles are always requested behind them (the path a late group takes).  For tests: which of the two
// paths a unit takes otherwise depends on timing.
bool never_early_for_test()
{
    const char *e = std::getenv("MYEA_LSTM_RESIDENT_TEST_NEVER_EARLY");
    return e && e[0] == '1';
}

// ---- host: the kernels on offer ------------------------------------------------------------------------------------------
using ResidentKernel = void (*)(ResidentGeometry, LstmResidentDir, LstmResidentDir, SyncWords);
struct KernelInfo {
    ResidentKernel fn = nullptr;
    size_t lds = 0;
    int cells = 0;
    int threads = kThreads;
    bool ready = false;
    hipError_t status = hipSuccess;
    int per_cu = 0;   // workgroups of this kernel a compute unit can hold
};

template <int KW, int CELLS, int RS, bool AGENT>
KernelInfo forward_info()
{
    KernelInfo k;
    k.fn = lstm_resident_forward_kernel<KW, CELLS, RS, AGENT>;
    k.lds = forward_lds(KW, CELLS, RS);
    k.cells = CELLS;
    return k;
}
template <int C, int RS>
KernelInfo backward_info()
{
    KernelInfo k;
    k.fn = lstm_resident_backward_kernel<C, RS>;
    k.lds = backward_lds(C, RS);
    k.cells = 16;
    return k;
}

template <int C>
KernelInfo sets_info()
{
    KernelInfo k;
    k.fn = lstm_resident_backward_sets_kernel<C>;
    k.lds = backward_sets_lds(C);
    k.cells = 16;
    k.threads = 2 * kThreads;
    return k;
}

template <int C>
KernelInfo ksplit_info()
{
    KernelInfo k;
    k.fn = lstm_resident_backward_ksplit_kernel<C>;
    k.lds = 0;   // its LDS is static
    k.cells = 16;
    return k;
}

// [backward][C: 128, 256, 512, 1024][rs - 1]; an entry without a kernel has fn == nullptr
KernelInfo g_kernels[2][4][2] = {
    {{forward_info<32, 16, 1, false>(), forward_info<32, 16, 2, false>()},
     {forward_info<64, 16, 1, false>(), forward_info<64, 16, 2, false>()},
     {forward_info<128, 16, 1, false>(), forward_info<128, 16, 2, false>()},
     {forward_info<256, 16, 1, true>(), KernelInfo{}}},
    {{backward_info<128, 1>(), backward_info<128, 2>()},
     {backward_info<256, 1>(), backward_info<256, 2>()},
     {backward_info<512, 1>(), KernelInfo{}},
     {backward_info<1024, 1>(), KernelInfo{}}},
};

// the backward loop split along k, [C: 128, 256, 512, 1024]: two chains of 16 examples only, groups within one XCD
KernelInfo g_ksplit[4] = {ksplit_info<128>(), ksplit_info<256>(), ksplit_info<512>(), KernelInfo{}};

// the backward loop with one chain per set of four wavefronts, [C: 128, 256, 512, 1024]: two chains of 16 examples, groups
// within one XCD
KernelInfo g_sets[4] = {KernelInfo{}, KernelInfo{}, sets_info<512>(), KernelInfo{}};

// MYEA_LSTM_BACKWARD_SETS=0 keeps the backward loop's two chains in one instruction stream
bool sets_disabled()
{
    const char *e = std::getenv("MYEA_LSTM_BACKWARD_SETS");
    return e && e[0] == '0';
}

// the kernel for (C, rs) with its LDS attribute set and its occupancy known, or nullptr
KernelInfo *kernel_for(size_t C, int rs, bool backward, bool ksplit = false, bool sets = false)
{
    const int ci = C == 128 ? 0 : C == 256 ? 1 : C == 512 ? 2 : C == 1024 ? 3 : -1;
    if (ci < 0 || rs < 1 || rs > 2 || ((ksplit || sets) && (rs != 1 || !backward))) return nullptr;
    KernelInfo &k = sets ? g_sets[ci] : ksplit ? g_ksplit[ci] : g_kernels[backward ? 1 : 0][ci][rs - 1];
    if (!k.fn) return nullptr;
    std::lock_guard<std::mutex> lock(g_resident_mutex);
    if (!k.ready) {
        k.status = k.lds ? hipFuncSetAttribute(reinterpret_cast<const void *>(k.fn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)k.lds) : hipSuccess;
        if (k.status == hipSuccess) k.status = hipOccupancyMaxActiveBlocksPerMultiprocessor(&k.per_cu, reinterpret_cast<const void *>(k.fn), k.threads, k.lds);
        k.ready = true;
    }
    return k.status == hipSuccess && k.per_cu >= 1 ? &k : nullptr;
}

// Groups of ROWS examples onto the device: LOCAL - an XCD hosts whole groups, as many as its compute units hold members;
// AGENT - the members of a group are spread over the device.  Every workgroup must be resident at once, or a wait between
// time steps could never end.
bool place_groups(const ResidentDevice &dev, const KernelInfo &k, int members, bool agent, int groups, int *grid)
{
    if (groups > kMaxGroups) return false;
    if (agent) { *grid = groups * members; return *grid <= dev.cus * k.per_cu; }
    const int per_xcd = (dev.cus / 8) * k.per_cu / members;   // groups one XCD can host
    const int slots = (groups + 7) / 8;                        // groups on the fullest XCD
    *grid = 8 * slots * members;
    return slots <= per_xcd;
}

int fill_geometry(const LstmResidentPlan &plan, size_t T, size_t B, size_t Bmax, size_t C, int dirs, ResidentGeometry *g)
{
    if (!plan.ok) { set_last_error("resident LSTM: no plan for this layer"); return MYEA_E_INVALID; }
    if (T < 2 || T > 0x7fffffffu / (unsigned)(plan.members + 1)) { set_last_error("resident LSTM: %zu time steps do not fit the barrier counters", T); return MYEA_E_INVALID; }
    g->T = (int)T; g->B = (int)B; g->Bmax = (int)Bmax; g->C = (int)C;
    g->dirs = dirs; g->row_groups = plan.row_groups; g->members = plan.members;
    g->arrivals = plan.members + (absent_member_for_test() ? 1 : 0);
    g->never_early = never_early_for_test() ? 1 : 0;
    g->spin_polls = spin_polls();
    return MYEA_OK;
}

// clears the counters and flags and lays the words out
int prepare_sync(hipStream_t s, const LstmResidentPlan &plan, int dirs, unsigned *sync, unsigned *host_flag, unsigned *fault, SyncWords *w)
{
    w->exchange = nullptr;
    const int groups = plan.row_groups * dirs;
    if (groups > kMaxGroups) { set_last_error("resident LSTM: %d groups exceed the counter block", groups); return MYEA_E_INVALID; }
    const int words = groups * 2 * kSyncStride + 1 + groups;
    hipLaunchKernelGGL(resident_clear_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, s, sync, words);
    MYEA_HIP_TRY(hipGetLastError());
    w->counters = sync;
    w->give_up = sync + (size_t)groups * 2 * kSyncStride;
    w->host_flag = host_flag;
    w->scrap = reinterpret_cast<float *>(sync + (size_t)kMaxGroups * 2 * kSyncStride + 1 + kMaxGroups);
    w->fault = fault ? fault : reinterpret_cast<unsigned *>(w->scrap);
    return MYEA_OK;
}

int check_dirs(const LstmResidentDir *dir, int dirs, bool backward)
{
    for (int k = 0; k < dirs; ++k) {
        const LstmResidentDir &d = dir[k];
        const bool fwd_ok = d.Wrec && d.bias && d.peep && d.acts && d.c && d.ca && d.h && !(reinterpret_cast<uintptr_t>(d.Wrec) & 15u) && !(reinterpret_cast<uintptr_t>(d.h) & 15u);
        const bool bwd_ok = d.WrecT && d.peep && d.acts && d.c && d.ca && d.dh && d.dG && d.dc && !(reinterpret_cast<uintptr_t>(d.WrecT) & 15u) && !(reinterpret_cast<uintptr_t>(d.dG) & 15u);
        if (backward ? !bwd_ok : !fwd_ok) { set_last_error("resident LSTM: null or unaligned operand"); return MYEA_E_INVALID; }
    }
    return MYEA_OK;
}

int launch_resident(hipStream_t s, bool backward, const LstmResidentPlan &plan, size_t T, size_t B, size_t Bmax, size_t C, int dirs,
                    const LstmResidentDir *dir, unsigned *sync, unsigned *host_flag, unsigned *fault, float *exchange = nullptr, size_t exchange_floats = 0)
{
    const bool ksplit = backward && plan.ksplit;
    ResidentGeometry g;
    SyncWords w;
    int rc = fill_geometry(plan, T, B, Bmax, C, dirs, &g);
    if (rc == MYEA_OK && backward && !plan.backward) { set_last_error("resident LSTM backward: no plan for this layer"); rc = MYEA_E_INVALID; }
    if (rc == MYEA_OK) rc = check_dirs(dir, dirs, backward);
    if (rc != MYEA_OK) return rc;
    if (ksplit) {
        for (int q = 0; q < dirs; ++q)
            if (!dir[q].Wrec) { set_last_error("resident LSTM backward: null operand"); return MYEA_E_INVALID; }
        const size_t need = lstm_resident_exchange_floats(C, B, dirs);
        if (!exchange || (reinterpret_cast<uintptr_t>(exchange) & 15u) || exchange_floats < need) {
            set_last_error("resident LSTM backward: the exchange buffer holds %zu floats, the layer needs %zu", exchange ? exchange_floats : (size_t)0, need);
            return MYEA_E_INVALID;
        }
    }
    KernelInfo *k = kernel_for(C, plan.rs, backward, ksplit);
    ResidentDevice *dev = nullptr;
    rc = probe_device(&dev);
    if (rc != MYEA_OK) return rc;
    int grid = 0;
    if (backward && !ksplit && !plan.agent && plan.rs == 1 && !sets_disabled() && dev->usable && (unsigned long long)T * Bmax * 4ull * C < (1ull << 30)) {   // its offsets are 32-bit byte counts
        // the column form with a set of wavefronts per chain, where it exists and maps onto the device like the plan's kernel
        KernelInfo *sets = kernel_for(C, plan.rs, true, false, true);
        if (sets && place_groups(*dev, *sets, plan.members, false, plan.row_groups * dirs, &grid) && grid == plan.grid) k = sets;
    }
    if (!k || !dev->usable || !place_groups(*dev, *k, plan.members, plan.agent, plan.row_groups * dirs, &grid) || grid != plan.grid) {
        set_last_error("resident LSTM: the plan does not fit the device (C = %zu, %d groups)", C, plan.row_groups * dirs);
        return MYEA_E_UNSUPPORTED;
    }
    rc = prepare_sync(s, plan, dirs, sync, host_flag, fault, &w);
    if (rc != MYEA_OK) return rc;
    w.exchange = ksplit ? exchange : nullptr;
    hipLaunchKernelGGL(k->fn, dim3((unsigned)plan.grid), dim3((unsigned)k->threads), k->lds, s, g, dir[0], dir[dirs > 1 ? 1 : 0], w);
    MYEA_HIP_TRY(hipGetLastError());
    return MYEA_OK;
}

}  // namespace

// How a layer of C cells (one per block) and B examples per direction maps onto the device, or plan.ok == false when the
// resident form does not apply (other widths, more examples than the device can hold groups for, probe failed).
// plan.backward: the backward loop has a resident form too (C <= 512).
int lstm_resident_plan(size_t C, size_t cells_per_block, size_t B, int dirs, LstmResidentPlan *plan)
{
    *plan = LstmResidentPlan{};
    if (resident_disabled() || cells_per_block != 1 || B == 0 || dirs < 1 || dirs > 2) return MYEA_OK;
    ResidentDevice *dev = nullptr;
    {
        const int rc = probe_device(&dev);
        if (rc != MYEA_OK) return rc;
    }
    if (!dev->usable) return MYEA_OK;
    // groups of two chains of 16 examples, or of 32 when there are more examples than the device holds such groups for
    for (int rs = 1; rs <= 2; ++rs) {
        KernelInfo *fwd = kernel_for(C, rs, false);
        if (!fwd) continue;
        KernelInfo *bwd = kernel_for(C, rs, true);
        const int members = (int)C / fwd->cells;
        const bool agent = members > dev->cus / 8;
        const int rows = 2 * 16 * rs, row_groups = (int)((B + rows - 1) / rows), groups = row_groups * dirs;
        int grid = 0, grid_b = 0;
        if (!place_groups(*dev, *fwd, members, agent, groups, &grid)) continue;
        // the backward kernel of 1024 cells is the device-scope one, the narrower ones keep a group on one XCD
        bool backward = bwd && agent == (C > 512) && place_groups(*dev, *bwd, members, agent, groups, &grid_b) && grid_b == grid;
        const int choice = ksplit_choice();
        KernelInfo *split = choice == 0 ? nullptr : kernel_for(C, rs, true, true);
        bool ksplit = split && !agent && fwd->cells == 16 && place_groups(*dev, *split, members, agent, groups, &grid_b) && grid_b == grid;
        const bool ksplit_available = ksplit;
        if (ksplit && backward && choice < 0) ksplit = 2 * groups * members <= dev->cus;
        backward = backward || ksplit;
        plan->ok = true; plan->agent = agent; plan->backward = backward; plan->ksplit = ksplit; plan->ksplit_available = ksplit_available && choice != 0;
        plan->cells = fwd->cells; plan->members = members; plan->rs = rs; plan->row_groups = row_groups; plan->grid = grid; plan->cus = dev->cus;
        break;
    }
    return MYEA_OK;
}

// Floats of exchange buffer the backward loop split along k needs for a layer of C cells and up to B examples per direction:
// per group of 32 examples and direction, 2 chains x 2 buffers x (C / 16)^2 tiles of 256 floats.  0 for other widths.
size_t lstm_resident_exchange_floats(size_t C, size_t B, int dirs)
{
    if ((C != 128 && C != 256 && C != 512) || B == 0 || dirs < 1) return 0;
    const size_t members = C / 16, groups = (B + 31) / 32 * (size_t)dirs;
    return groups * 4 * members * members * 256;
}

// counters (one per group and chain, 128 bytes apart), the give-up flag, one XCC word per group, the scrap area
size_t lstm_resident_sync_words() { return (size_t)kMaxGroups * 2 * kSyncStride + 1 + kMaxGroups + kScrapWords; }

// sync: lstm_resident_sync_words() unsigneds of device memory (cleared by the call); host_flag: one pinned host word (0 = fine)
int launch_lstm_resident_forward(hipStream_t s, const LstmResidentPlan &plan, size_t T, size_t B, size_t Bmax, size_t C, int dirs,
                                 const LstmResidentDir *dir, unsigned *sync, unsigned *host_flag, unsigned *fault)
{
    return launch_resident(s, false, plan, T, B, Bmax, C, dirs, dir, sync, host_flag, fault);
}

int launch_lstm_resident_backward(hipStream_t s, const LstmResidentPlan &plan, size_t T, size_t B, size_t Bmax, size_t C, int dirs,
                                  const LstmResidentDir *dir, unsigned *sync, unsigned *host_flag, unsigned *fault, float *exchange, size_t exchange_floats)
{
    return launch_resident(s, true, plan, T, B, Bmax, C, dirs, dir, sync, host_flag, fault, exchange, exchange_floats);
}

}  // namespace myea
