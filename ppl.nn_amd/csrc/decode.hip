// Decode attention over the int8 group-8 KV slab (one new token per sequence, which the kernel also quantises into
// the slab), split along the cached tokens.
//
// Roofline: HBM. Each cached token costs 2 * KVH * (Dh + Dh/4) bytes and is read exactly once; arithmetic
// intensity is 1.6 .. 12.8 flop/B. Three things have to stay below the HBM time for the kernel to sit on that
// roofline: vector-ALU work (dequantisation), matrix-core work, and the number of vector-memory instructions the
// texture addresser has to walk through. The design answers each:
//   * Bytes travel global -> LDS with global_load_lds_dwordx4 (no registers, 16 B per lane, every instruction covers
//     whole 128 B rows of the slab), ten instructions per 32 tokens instead of two dozen narrow gathers.
//   * Each wave stages its own tokens in its own LDS region, double buffered: the DMA of the next 32 tokens is in
//     flight while the current 32 are computed. Only wave-level waits are needed, no workgroup barriers.
//   * All H/KVH query heads of a kv head ride in the 16-wide N dimension of v_mfma_f32_16x16x32_f16, so a KV byte is
//     read once whatever the grouping, and the contraction costs two dozen MFMAs per 32 tokens.
//
// Work decomposition (balanced on the device, no host knowledge of the lengths): the cached tokens of all decode
// sequences, laid end to end (kvstarts is exactly that prefix sum), are cut into S ranges of equal cost (equal length
// on an axis that charges every sequence boundary a few positions: see kBoundaryTokens). One workgroup owns one
// range for a group of up to 4 kv heads; where its range crosses sequence boundaries it handles the pieces ("segments")
// one after the other. Every workgroup therefore streams the same number of bytes, whatever the raggedness of the batch,
// and there is no tail of long sequences. Inside a workgroup each wave owns one kv head (the workgroup then reads
// hpb * 128 contiguous bytes of every token) or, with fewer than 4 kv heads, a share of the segment's tokens.
// The head groups of one range are neighbouring workgroups: they start together and reach the same DRAM pages together.
//
// LDS layout of one 32-token stage of one wave (10 KiB): K rows [32][128 B], V rows [32][128 B], K scales [32][32 B],
// V scales [32][32 B]. Inside a K/V row the eight 16 B pieces are XOR-swizzled with (row & 7) by choosing which
// global piece each DMA lane fetches, so the MFMA-layout reads below (16 different rows per instruction) spread over
// all banks.
//
// Per 16-token block a lane (m = lane & 15, kq = lane >> 4) does:
//   S^T = K_hat * Q^T   A = K_hat[token m][channels 32*kq + 16*j + 8*i .. +7]  (two ds_read_b128, one scale b64 per lane)
//                       B = Q^T, held in registers for the whole task
//         -> lane holds scores of head m for tokens 4*kq .. 4*kq+3
//   O^T += V_hat^T * P^T  A = V_hat^T[channel 8*m + i][tokens 4*kq .. +3]  (four ds_read_b64 per lane, transposed in
//                       registers with v_perm), B = P^T straight from the score registers
// int8 -> fp16 is exact: (x ^ 0x80) placed under exponent byte 0x64 reads as 1024 + (x + 128); subtract 1152, then
// multiply by the group's fp16 scale (packed fp16 ops). Softmax runs online in the exp2 domain with fp32 statistics.
//
// A segment that is a whole sequence is normalised and written as fp16 output directly. Otherwise the workgroup writes
// one un-normalised partial (max, sum, acc[Dh]) per query head into workspace slot (range index + sequence index) --
// consecutive (range, sequence) segments get consecutive slots -- and `decode_merge_kernel` combines the slots of a
// sequence with the usual log-sum-exp weights.
#include <atomic>
#include <initializer_list>
#include <type_traits>
#include "common.h"

namespace pplhip {

constexpr int kDh = 128; // head_dim this kernel is specialised for
constexpr int kDecodeWaves = 4; // waves per workgroup; each owns a 20 KiB double-buffered LDS region
constexpr int kStageTokens = 32; // tokens per pipeline stage (2 MFMA sub-blocks of 16)
constexpr int kSubBlocks = kStageTokens / 16;
// LDS bytes of one stage of one wave, and where its four arrays start
constexpr int kLdsK = 0;
constexpr int kLdsV = kStageTokens * 128;
constexpr int kLdsKs = 2 * kStageTokens * 128;
constexpr int kLdsVs = kLdsKs + kStageTokens * 32;
constexpr int kStageBytes = kLdsVs + kStageTokens * 32; // 10240
constexpr int kWaveLdsBytes = 2 * kStageBytes;
constexpr int kDecodeLdsBytes = kDecodeWaves * kWaveLdsBytes; // 81920: two workgroups fill a CU's 160 KiB

struct DecodeParams {
    const half_t* q; // [S, H, Dh]
    const half_t* cur_key; // [S, KVH, Dh] new tokens: the decode sequences' are quantised into the slab by this launch
    const half_t* cur_value;
    int8_t* cache;
    half_t* scale;
    const int64_t* seqstarts;
    const int64_t* kvstarts;
    const int64_t* cachestarts; // [nd], or the [nd, cs_stride_b] page table when page_shift > 0
    int64_t cs_stride_b;
    int32_t page_shift; // 0: contiguous region per sequence; else pages of 2^page_shift tokens
    half_t* out; // [S, H, Dh]
    float* part_acc; // [slots, H, Dh], slots = num_ranges + nd
    float* part_ml; // [slots, H, 2]
    int32_t* range_first; // [num_ranges] first sequence of every range, written by the decode kernel for the merge
    CacheAddr addr;
    int32_t nd; // decode sequences (the first nd entries of the tables)
    int32_t num_heads, kv_heads, rep; // rep = num_heads / kv_heads (<= 16)
    int32_t num_ranges; // S
    int32_t hpb; // kv heads per workgroup: min(kv_heads, 4), a power of two dividing kv_heads
    int32_t merge_by_boundary; // merge kernel: blockIdx.y counts range boundaries instead of sequences
    // Head dims 64 and 32: 2 (4) kv heads that lie next to each other in the slab are streamed as ONE kv head of 128
    // channels ("virtual" head: kv_heads, rep and addr.stride_h above are the virtual ones, rep = 2 (4) x the real
    // number of query heads per kv head, at most 16). A query head's 64 (32) channels sit in its own part of the
    // 128-channel query operand, zeros elsewhere, so its scores come out of the other heads' channels as + 0; of its
    // 128 output channels only its own part means anything and is stored. sub_shift = log2(128 / head_dim): 0, 1, 2.
    int32_t sub_shift;
    int32_t new_tokens_written_elsewhere; // the launch's write-only workgroups put the decode sequences' new tokens
                                          // into the slab: the decode waves only patch their stage buffers
    float score_scale; // log2(e) / sqrt(Dh)
};

// Every sequence boundary inside a range costs the range's workgroup about one stage more (the sequence before the
// boundary ends with a partly filled stage, the one behind it starts a new one), and the launch lasts as long as the
// range with the most boundaries. The ranges are therefore cut on a virtual axis on which every sequence is followed by
// kBoundaryTokens positions that hold no token: sequence i starts at kvstarts[i] + i * kBoundaryTokens. Equal virtual
// ranges give a range with many boundaries fewer tokens.
constexpr int kBoundaryTokens = 32;

// a / b for non-negative a and positive b: positions are nearly always below 2^32, and a 32-bit division is a fraction
// of the 64-bit one's instructions (neither has hardware behind it)
__device__ inline int64_t div_positions(int64_t a, int64_t b) {
    if (((uint64_t)a | (uint64_t)b) >> 32) return a / b;
    return (int64_t)((uint32_t)a / (uint32_t)b);
}

// Positions per range: the total is only known on the device. At least 128 so that tiny batches are not shredded.
__device__ inline int64_t range_tokens(int64_t total, int num_ranges) {
    int64_t r = div_positions(total + num_ranges - 1, num_ranges);
    r = (r + 31) & ~(int64_t)31;
    return r < 128 ? 128 : r;
}

// The sequence tables are read through the constant address space: a wave-uniform read from there is always a scalar
// load. Through a plain global pointer the compiler only uses scalar loads while the kernel has not stored anything;
// after the first result store the look-ups of the next sequence became vector loads, whose result is only there
// once every transfer in flight has landed (one counter, in order): each sequence boundary drained the pipeline.
typedef const int64_t __attribute__((address_space(4)))* const_tab_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

// Reductions over the four 16-lane rows of the wave (lanes l, l^16, l^32, l^48) in the vector ALU: the swap
// instructions hand every lane of a row pair both rows' values, where a shuffle would be a round trip through the LDS
// pipeline. v_permlane16_swap(x, y) exchanges the odd rows of x with the even rows of y; v_permlane32_swap(x, y) the
// upper half of x with the lower half of y; with x = y = v the two results hold the two partners' values.
__device__ inline float wave_max_over_quads(float v) {
    const uint32_t u = __float_as_uint(v);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const uint32_t w = __float_as_uint(v);
    const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ inline float wave_sum_over_quads(float v) {
    const uint32_t u = __float_as_uint(v);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const uint32_t w = __float_as_uint(v);
    const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Pins a pointer that is wave-uniform by construction into scalar registers, so that memory instructions take the
// "scalar base + 32-bit lane offset" addressing form.
__device__ inline const char* make_uniform(const char* p) {
    const uint64_t u = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
    return reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
}

// LDS reads of DMA-filled buffers go through inline assembly: for compiler-visible LDS loads the waitcnt pass cannot
// tell which DMA transfer they depend on and drains ALL outstanding transfers first (vmcnt(0)), which would serialise
// the pipeline. Here the ordering is explicit: PPLHIP_WAIT_VMCNT before the first read of a stage, and
// PPLHIP_WAIT_LGKMCNT + a scheduling barrier before the first use of the values read.
template <int OFF>
__device__ inline uint4 lds_read_b128(uint32_t addr) {
    uint4 r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
}
template <int OFF>
__device__ inline uint2 lds_read_b64(uint32_t addr) {
    uint2 r;
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
}
template <int OFF>
__device__ inline uint32_t lds_read_u16(uint32_t addr) {
    uint32_t r;
    asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
}
// LDS stores the compiler does not see either: a visible LDS access makes it wait for every transfer in flight
__device__ inline void lds_write_b64(uint32_t addr, uint2 v) {
    asm volatile("ds_write_b64 %0, %1" ::"v"(addr), "v"(v) : "memory");
}
__device__ inline void lds_write_b16(uint32_t addr, uint32_t v) {
    asm volatile("ds_write_b16 %0, %1" ::"v"(addr), "v"(v) : "memory");
}
#define PPLHIP_WAIT_LGKMCNT(n)                                  \
    do {                                                        \
        asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(n) : "memory"); \
        __builtin_amdgcn_sched_barrier(0);                      \
    } while (0)

// s_waitcnt vmcnt(n) only (expcnt / lgkmcnt left at "no wait"), gfx9 encoding
#define PPLHIP_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xf) | (((n) >> 4) << 14) | 0x0f70)
// the same with `extra` (0, 4 or 8: result stores of the previous segment) younger operations more left in flight; the
// immediate has to be a constant.
// These counts are kept by hand: `n` is the number of transfers and untracked loads issued after the data that is
// waited for, `extra` a lower bound on the store instructions issued after those. A build with
// -DPPLHIP_CONSERVATIVE_WAITS waits for everything in flight instead (slower, no counting to get wrong); its results
// must be bit-identical, which is what a test of the two builds against each other checks.
#ifdef PPLHIP_CONSERVATIVE_WAITS
#define PPLHIP_WAIT_VMCNT_PLUS(n, extra) \
    do {                                 \
        (void)(extra);                   \
        PPLHIP_WAIT_VMCNT(0);            \
    } while (0)
#else
#define PPLHIP_WAIT_VMCNT_PLUS(n, extra)            \
    do {                                            \
        switch (extra) {                            \
            case 4: PPLHIP_WAIT_VMCNT((n) + 4); break; \
            case 8: PPLHIP_WAIT_VMCNT((n) + 8); break; \
            default: PPLHIP_WAIT_VMCNT(n); break;      \
        }                                           \
    } while (0)
#endif
// A 16-byte global load the compiler does not track: its waitcnt pass merges what it knows about loads in flight at
// every loop header, and for the query registers (loaded once per sequence, read by every stage) that put a
// vmcnt(0) in front of the first MFMA of EVERY stage and another in front of every stage's transfers -- the wave never
// computed while one of its own transfers was in flight. The waits for these loads are the explicit ones in the
// stage loop (they are older than the stage they are used with) and the one in front of the hand-over to the next
// segment. The destination must be the variable the value lives in until such a wait: a copy made earlier would copy
// registers the data has not reached.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
// and must not be carried around a loop before that wait (the copies of a loop-carried value are made at once).
__device__ inline void load16_untracked(half8_t& dst, const void* ptr) {
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(ptr) : "memory");
}
__device__ inline void load16_untracked(u32x4_t& dst, const void* ptr) {
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(ptr) : "memory");
}
constexpr int kDmaPerStage = 2 * (kStageTokens / 8) + 2; // 4 K + 4 V + K scales + V scales

// Per-lane source offsets of the stage DMA (relative to the wave-uniform stage base).
struct DmaOffsets {
    uint32_t kv[kStageTokens / 8]; // rows 8*i + lane/8: row * stride + swizzled piece * 16
    uint32_t sc; // row lane/2: row * scale stride + (lane & 1) * 16
    uint8_t kv_row[kStageTokens / 8], sc_row; // the (clamped) rows themselves: the paged path picks a page per row
};

// rows_mem: rows of the stage that exist in the chunk (1..32); later rows are clamped onto the last one
__device__ inline void make_dma_offsets(DmaOffsets& o, int lane, uint32_t stride, uint32_t sstride_b, int rows_mem) {
    const int piece = (lane & 7) ^ (lane >> 3); // LDS slot (lane & 7) of row r holds global piece slot ^ (r & 7)
#pragma unroll
    for (int i = 0; i < kStageTokens / 8; ++i) {
        int r = 8 * i + (lane >> 3);
        r = r < rows_mem ? r : rows_mem - 1;
        // the swizzle key is the LDS row (8*i + lane/8) & 7 = lane >> 3, whatever row the bytes come from
        o.kv[i] = (uint32_t)r * stride + 16u * piece;
        o.kv_row[i] = (uint8_t)r;
    }
    int rs = lane >> 1;
    rs = rs < rows_mem ? rs : rows_mem - 1;
    o.sc = (uint32_t)rs * sstride_b + 16u * (lane & 1);
    o.sc_row = (uint8_t)rs;
}

// Cache policy of the K/V row transfers: the `nt` (non-temporal) bit. Every int8 row is read exactly once per call and
// is a whole 128-byte cache line, so nothing is gained by keeping it in L2, and the streaming policy is worth a
// fifth of the bandwidth: a bare loop of the same transfers streams 6.2 TB/s without the bit and 7.0 TB/s with it, the
// kernel 64.3 -> 69.5 % of 8 TB/s on 120 x 32-kv-head-group sequences. The scale rows keep the default policy: the four
// waves of a workgroup (four kv heads) each fetch 32 bytes of the same 128-byte line per token, and with `nt` every one
// of them went to memory on its own (measured: 59.5 %).
constexpr int kStreamOnce = 2; // aux / cache-policy operand of global_load_lds: bit 1 = nt

// Enqueues the 10 global->LDS transfers of one stage. cbase/sbase: K row 0 of the stage in the cache / scale tensors;
// kv_off / kv_off_s: distance from a K row to the V row of the same token.
__device__ inline void dma_stage(char* lds_stage, const char* cbase, const char* sbase, const DmaOffsets& o,
                                 int64_t kv_off, int64_t kv_off_s) {
    // the K -> V distance is folded into the wave-uniform base (it exceeds 32 bits in a large cache_layout 3 slab)
    const char* vbase = cbase + kv_off;
    const char* vsbase = sbase + kv_off_s;
#pragma unroll
    for (int i = 0; i < kStageTokens / 8; ++i) {
        __builtin_amdgcn_global_load_lds((gbl_ptr_t)(cbase + o.kv[i]), (lds_ptr_t)(lds_stage + kLdsK + 1024 * i), 16, 0,
                                         kStreamOnce);
        __builtin_amdgcn_global_load_lds((gbl_ptr_t)(vbase + o.kv[i]), (lds_ptr_t)(lds_stage + kLdsV + 1024 * i), 16, 0,
                                         kStreamOnce);
    }
    __builtin_amdgcn_global_load_lds((gbl_ptr_t)(sbase + o.sc), (lds_ptr_t)(lds_stage + kLdsKs), 16, 0, 0);
    __builtin_amdgcn_global_load_lds((gbl_ptr_t)(vsbase + o.sc), (lds_ptr_t)(lds_stage + kLdsVs), 16, 0, 0);
}

// The same 10 transfers when a stage may straddle two pages of a paged slab: rows below `split` come from page A
// (cbase_a / sbase_a address row 0 of the stage), the others from page B (cbase_b / sbase_b address the row that
// would precede page B's first row by `split` rows, so the same per-row offsets apply). The base is then per lane,
// so these transfers take the 64-bit vector-address form.
__device__ inline void dma_stage_paged(char* lds_stage, const char* cbase_a, const char* cbase_b, const char* sbase_a,
                                       const char* sbase_b, int split, const DmaOffsets& o, int64_t kv_off,
                                       int64_t kv_off_s) {
#pragma unroll
    for (int i = 0; i < kStageTokens / 8; ++i) {
        const char* cb = (o.kv_row[i] < split ? cbase_a : cbase_b) + o.kv[i];
        __builtin_amdgcn_global_load_lds((gbl_ptr_t)cb, (lds_ptr_t)(lds_stage + kLdsK + 1024 * i), 16, 0, kStreamOnce);
        __builtin_amdgcn_global_load_lds((gbl_ptr_t)(cb + kv_off), (lds_ptr_t)(lds_stage + kLdsV + 1024 * i), 16, 0,
                                         kStreamOnce);
    }
    const char* sb = (o.sc_row < split ? sbase_a : sbase_b) + o.sc;
    __builtin_amdgcn_global_load_lds((gbl_ptr_t)sb, (lds_ptr_t)(lds_stage + kLdsKs), 16, 0, 0);
    __builtin_amdgcn_global_load_lds((gbl_ptr_t)(sb + kv_off_s), (lds_ptr_t)(lds_stage + kLdsVs), 16, 0, 0);
}

// Per-lane LDS read offsets inside a stage (they are the same for every stage).
struct ReadOffsets {
    uint32_t k[2]; // K row m, pieces 2*kq and 2*kq + 1 (swizzled)      (+2048 per sub-block)
    uint32_t ks; // K scale row m, groups 4*kq .. 4*kq + 3              (+512 per sub-block)
    uint32_t v[4]; // V row 4*kq + e, 8 channels of group m (swizzled)   (+2048 per sub-block)
    uint32_t vs; // V scale row 4*kq, group m                           (+32 per e, +512 per sub-block)
};

__device__ inline void make_read_offsets(ReadOffsets& r, int m, int kq) {
#pragma unroll
    for (int j = 0; j < 2; ++j) r.k[j] = kLdsK + m * 128 + (((2 * kq + j) ^ (m & 7)) * 16);
    r.ks = kLdsKs + m * 32 + kq * 8;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int row = 4 * kq + e;
        r.v[e] = kLdsV + row * 128 + (((m >> 1) ^ (row & 7)) * 16) + (m & 1) * 8;
    }
    r.vs = kLdsVs + (4 * kq) * 32 + m * 2;
}

struct SoftmaxState {
    float4_t oacc[8]; // O^T: oacc[i][e] = channel 8*(4*kq + e) + i of head m
    float m_run; // running max of head m in the exp2 domain (same in the 4 lanes that share m)
    float l_part; // this lane's share of the running sum
};

template <int SB>
__device__ inline void read_stage_sub(uint4 (&kr)[2], uint2& ksr, uint2 (&vr)[4], uint32_t (&vsr)[4], const uint32_t (&ak)[2],
                                      uint32_t aks, const uint32_t (&av)[4], uint32_t avs) {
    kr[0] = lds_read_b128<2048 * SB>(ak[0]);
    kr[1] = lds_read_b128<2048 * SB>(ak[1]);
    ksr = lds_read_b64<512 * SB>(aks);
    vr[0] = lds_read_b64<2048 * SB>(av[0]);
    vr[1] = lds_read_b64<2048 * SB>(av[1]);
    vr[2] = lds_read_b64<2048 * SB>(av[2]);
    vr[3] = lds_read_b64<2048 * SB>(av[3]);
    vsr[0] = lds_read_u16<512 * SB + 0>(avs);
    vsr[1] = lds_read_u16<512 * SB + 32>(avs);
    vsr[2] = lds_read_u16<512 * SB + 64>(avs);
    vsr[3] = lds_read_u16<512 * SB + 96>(avs);
}

// lds_stage: LDS byte address of the stage buffer. rows_valid: tokens of this stage that belong to the wave's range
// (1..32); the rest is masked out of the softmax.
template <typename AfterReads>
__device__ inline void compute_stage(uint32_t lds_stage, const ReadOffsets& ro, SoftmaxState& ss,
                                     const half8_t (&qB)[2][2], int kq, int rows_valid, float score_scale,
                                     AfterReads&& after_reads) {
    static_assert(kSubBlocks == 2, "the stage is processed as two 16-token sub-blocks");
    const uint32_t ak[2] = {ro.k[0] + lds_stage, ro.k[1] + lds_stage};
    const uint32_t aks = ro.ks + lds_stage, avs = ro.vs + lds_stage;
    const uint32_t av[4] = {ro.v[0] + lds_stage, ro.v[1] + lds_stage, ro.v[2] + lds_stage, ro.v[3] + lds_stage};
    uint4 kr[kSubBlocks][2];
    uint2 ksr[kSubBlocks];
    uint2 vraw[kSubBlocks][4];
    uint32_t vsr[kSubBlocks][4];
    read_stage_sub<0>(kr[0], ksr[0], vraw[0], vsr[0], ak, aks, av, avs);
    read_stage_sub<1>(kr[1], ksr[1], vraw[1], vsr[1], ak, aks, av, avs);
    PPLHIP_WAIT_LGKMCNT(0);
    // the stage now lives in registers: its buffer may take the transfers of a later stage while the arithmetic runs
    after_reads();
    __builtin_amdgcn_sched_barrier(0);

    // ---- scores S^T[token, head]: v_mfma_f32_16x16x32_f16, one quantisation group (8 channels) per lane per MFMA
    float4_t sc[kSubBlocks];
#pragma unroll
    for (int sb = 0; sb < kSubBlocks; ++sb) {
        float4_t acc = {0.f, 0.f, 0.f, 0.f};
        const half2_t s01 = as_half2(ksr[sb].x), s23 = as_half2(ksr[sb].y);
        const half_t gs[4] = {s01.x, s01.y, s23.x, s23.y};
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const half8_t a0 = dequant8(kr[sb][j].x, kr[sb][j].y, gs[2 * j]);
            const half8_t a1 = dequant8(kr[sb][j].z, kr[sb][j].w, gs[2 * j + 1]);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, qB[j][0], acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, qB[j][1], acc, 0, 0, 0);
        }
        // lane now holds head m, tokens 16*sb + 4*kq + e of the stage
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = (16 * sb + 4 * kq + e < rows_valid) ? acc[e] * score_scale : -INFINITY;
        sc[sb] = acc;
    }
    // ---- online softmax update (per head = per lane column m)
    float mx = -INFINITY;
#pragma unroll
    for (int sb = 0; sb < kSubBlocks; ++sb)
#pragma unroll
        for (int e = 0; e < 4; ++e) mx = fmaxf(mx, sc[sb][e]);
    mx = wave_max_over_quads(mx);
    const float m_new = fmaxf(ss.m_run, mx); // finite: the first token of every computed stage is valid
    const float alpha = __builtin_amdgcn_exp2f(ss.m_run - m_new);
    ss.m_run = m_new;
    float psum = 0.f;
    float pe[kSubBlocks][4];
#pragma unroll
    for (int sb = 0; sb < kSubBlocks; ++sb)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            pe[sb][e] = __builtin_amdgcn_exp2f(sc[sb][e] - m_new);
            psum += pe[sb][e];
        }
    // B operand of the PV product: k-slot e8 of this lane <-> token 16*(e8/4) + 4*kq + e8%4 of the stage
    const half8_t pB = {(half_t)pe[0][0], (half_t)pe[0][1], (half_t)pe[0][2], (half_t)pe[0][3],
                        (half_t)pe[1][0], (half_t)pe[1][1], (half_t)pe[1][2], (half_t)pe[1][3]};
    ss.l_part = ss.l_part * alpha + psum;
    if (__any(alpha != 1.0f)) { // once the running maxima have settled, the rescale is skipped (wave-uniform branch)
#pragma unroll
        for (int i = 0; i < 8; ++i) ss.oacc[i] *= alpha;
    }
    // ---- O^T[channel, head] += V_hat^T * P^T over the stage's 32 tokens: one 16x16x32 MFMA per channel i
    half2_t vs2[kSubBlocks][4];
#pragma unroll
    for (int sb = 0; sb < kSubBlocks; ++sb)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t dup = vsr[sb][e] | (vsr[sb][e] << 16);
            vs2[sb][e] = as_half2(dup);
        }
#pragma unroll
    for (int cp = 0; cp < 4; ++cp) { // channel pair 8*m + 2*cp, 2*cp + 1 of this lane
        half2_t d[kSubBlocks][4]; // dequantised [sb][token e]
#pragma unroll
        for (int sb = 0; sb < kSubBlocks; ++sb)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t x = ((cp < 2) ? vraw[sb][e].x : vraw[sb][e].y) ^ 0x80808080u;
                d[sb][e] = dequant2((cp & 1) ? widen_hi(x) : widen_lo(x), vs2[sb][e]);
            }
#pragma unroll
        for (int odd = 0; odd < 2; ++odd) {
            const uint32_t sel = odd ? 0x07060302u : 0x05040100u;
            uint32_t t[4];
#pragma unroll
            for (int sb = 0; sb < kSubBlocks; ++sb) {
                t[2 * sb + 0] = __builtin_amdgcn_perm(as_u32(d[sb][1]), as_u32(d[sb][0]), sel);
                t[2 * sb + 1] = __builtin_amdgcn_perm(as_u32(d[sb][3]), as_u32(d[sb][2]), sel);
            }
            half8_t a;
            __builtin_memcpy(&a, t, 16);
            const int i = 2 * cp + odd;
            ss.oacc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pB, ss.oacc[i], 0, 0, 0);
        }
    }
}

// The wave that owns the tail of a sequence quantises the sequence's new token into the slab (and into its stage
// buffer) itself.
// DIRECT: every wave owns a whole kv head (hpb == waves per workgroup); otherwise the waves split the tokens of a kv
// head and combine through LDS.
// `block`: the workgroup's index among the decode workgroups of the launch (they come first in the grid); `smem`: the
// launch's dynamic LDS, kDecodeLdsBytes of it.
template <bool PAGED, bool DIRECT>
__device__ __forceinline__ void decode_workgroup(const DecodeParams& p, uint32_t block, char* smem) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // wave-uniform by construction
    const int groups = p.kv_heads / p.hpb;
    // Workgroup numbering: the head groups of a range are neighbours. (Numbering them so that they share an XCD, with
    // the range count rounded down to a multiple of 8 for it, measured the same on every shape -- the head groups read
    // different bytes of a row, there is nothing for them to share in an L2 -- and left up to 7 x groups slots empty.)
    const int hg = (int)(block % (uint32_t)groups);
    const int64_t s_idx = block / (uint32_t)groups; // range index
    // (virtual positions: see kBoundaryTokens)
    const const_tab_t kvstarts = (const_tab_t)p.kvstarts, seqstarts = (const_tab_t)p.seqstarts,
                      cachestarts = (const_tab_t)p.cachestarts;
    const int64_t total = kvstarts[p.nd] + (int64_t)p.nd * kBoundaryTokens;
    const int64_t R = range_tokens(total, p.num_ranges);
    const int64_t r0 = s_idx * R;
    if (r0 >= total) return;
    const int64_t r1 = (r0 + R < total) ? r0 + R : total;

    const int kvh_local = wave & (p.hpb - 1);
    const int kvh = hg * p.hpb + kvh_local;
    const int tsplits = DIRECT ? 1 : kDecodeWaves / p.hpb;
    const int ts = DIRECT ? 0 : wave / p.hpb;
    const int m = lane & 15;
    const int kq = lane >> 4;

    // bytes between tokens (int8 elements); the entry points reject strides of 2^25 and more, so the offsets of a
    // 32-token stage (and of a 64-token prefill tile) fit 32 bits
    const uint32_t stride = (uint32_t)p.addr.stride_s;
    const uint32_t sstride_b = (uint32_t)(p.addr.stride_s / kQuantGroup) * 2u;
    const int64_t kv_off = p.addr.stride_kv; // up to KVH * MaxT * Dh in cache_layout 3: not a 32-bit quantity
    const int64_t kv_off_s = p.addr.stride_kv / kQuantGroup * 2;
    const int64_t step_c = (int64_t)kStageTokens * stride, step_s = (int64_t)kStageTokens * sstride_b;
    DmaOffsets full;
    make_dma_offsets(full, lane, stride, sstride_b, kStageTokens);
    ReadOffsets ro;
    make_read_offsets(ro, m, kq);
    char* wave_lds = smem + wave * kWaveLdsBytes;
    const uint32_t wave_lds_addr =
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem + wave * kWaveLdsBytes;
    float* lds = reinterpret_cast<float*>(smem);
    const int row_f = kDh + 2;

    // First sequence of the range: count the sequences that end at or before r0. One coalesced vector load per 64
    // table entries and a ballot, instead of a binary search whose scalar loads would each wait for the previous one.
    int b = 0;
    for (int base = 0; base < p.nd; base += kWave) {
        const int i = base + lane;
        const bool ends_before = i < p.nd && p.kvstarts[i + 1] + (int64_t)(i + 1) * kBoundaryTokens <= r0;
        b += __builtin_popcountll(__ballot(ends_before));
    }
    b = __builtin_amdgcn_readfirstlane(b);
    if (hg == 0 && threadIdx.x == 0) p.range_first[s_idx] = b; // saves the merge kernel the same search
    int64_t pos = r0;
    if (r0 - (kvstarts[b] + (int64_t)b * kBoundaryTokens) >= kvstarts[b + 1] - kvstarts[b]) {
        // the range starts in the empty positions behind sequence b: its first token is the next sequence's first
        ++b;
        if (b >= p.nd) return;
        pos = kvstarts[b] + (int64_t)b * kBoundaryTokens;
        if (pos >= r1) return;
    }

    // A segment = the part of one sequence inside this range; this wave's share of it is tokens [t_begin, t_end).
    struct Segment {
        int b;
        int32_t seg_end, qrow, t_begin; // positions inside a sequence and packed token rows fit 32 bits
        bool whole_sequence;
        const_tab_t page_row; // paged slab: the sequence's row of the page table
        const char* cbase; // contiguous slab: K row of token t_begin (this kv head) in the cache tensor
        int n_stages, tail_rows_mem, tail_rows_valid;
        // this wave's chunk ends with the sequence's NEW token (its last one), which the wave quantises into the slab
        // and into its stage buffer itself
        bool has_new;
    };
    const int64_t head_off = p.addr.row(0, 0, kvh); // layer and kv head, K plane
    auto next_segment = [&](Segment& g) { // consumes sequence b from (virtual) position pos on
        const int64_t seq_lo = kvstarts[b], seq_hi = kvstarts[b + 1];
        const int64_t vlo = seq_lo + (int64_t)b * kBoundaryTokens; // virtual position of the sequence's first token
        const int64_t seg_begin = pos - vlo; // < the sequence's length
        g.b = b;
        g.seg_end = (int32_t)((r1 - vlo < seq_hi - seq_lo) ? r1 - vlo : seq_hi - seq_lo);
        g.whole_sequence = seg_begin == 0 && g.seg_end == seq_hi - seq_lo;
        g.page_row = PAGED ? cachestarts + (int64_t)b * p.cs_stride_b : nullptr;
        g.qrow = (int32_t)seqstarts[b];
        // (tsplits is 1, 2 or 4; a segment's length fits 32 bits)
        int64_t sub = (int64_t)((uint32_t)(g.seg_end - seg_begin + tsplits - 1) / (uint32_t)tsplits);
        sub = (sub + kStageTokens - 1) / kStageTokens * kStageTokens;
        g.t_begin = (int32_t)(seg_begin + (int64_t)ts * sub);
        const int64_t t_end = (g.t_begin + sub < g.seg_end) ? g.t_begin + sub : (int64_t)g.seg_end; // may be <= t_begin: none
        g.n_stages = t_end > g.t_begin ? (int)((t_end - g.t_begin + kStageTokens - 1) / kStageTokens) : 0;
        // The wave's last stage may overhang: rows past the end of the SEGMENT are clamped onto its last row (loads
        // must stay inside memory the sequence owns) and everything past the wave's own range is masked.
        const int64_t last_stage_t0 = g.t_begin + (int64_t)(g.n_stages - 1) * kStageTokens;
        g.tail_rows_mem =
            (int)(((int64_t)g.seg_end - last_stage_t0) < kStageTokens ? ((int64_t)g.seg_end - last_stage_t0) : kStageTokens);
        g.tail_rows_valid = (int)(t_end - last_stage_t0);
        g.has_new = g.n_stages > 0 && t_end == seq_hi - seq_lo;
        const int64_t row0 = (PAGED ? 0 : (cachestarts[b] + (int64_t)g.t_begin) * (int64_t)stride) + head_off;
        g.cbase = reinterpret_cast<const char*>(p.cache) + row0;
        // where the range goes on: inside this sequence (then pos = r1), or at the next sequence's first token
        pos = vlo + g.seg_end + (g.seg_end == seq_hi - seq_lo ? kBoundaryTokens : 0);
        ++b;
    };
    // enqueues stage idx of segment g into stage buffer `slot`
    auto issue_with = [&](const Segment& g, int idx, int slot, const DmaOffsets& off, int rows_mem) {
        char* dst = wave_lds + slot * kStageBytes;
        if (PAGED) {
            // a stage of 32 tokens touches at most two pages (pages hold >= 64 tokens)
            const int64_t t0 = (int64_t)g.t_begin + (int64_t)idx * kStageTokens;
            const int64_t in_page = t0 & ((int64_t(1) << p.page_shift) - 1);
            const int64_t left = (int64_t(1) << p.page_shift) - in_page; // rows of the stage in its first page
            const int split = left < kStageTokens ? (int)left : kStageTokens;
            const int64_t pa = g.page_row[t0 >> p.page_shift];
            // the second page exists whenever one of the stage's (clamped) rows lies in it
            const int64_t pb = split < rows_mem ? g.page_row[(t0 >> p.page_shift) + 1] : pa;
            const int64_t ra = (pa + in_page) * (int64_t)stride + head_off;
            const int64_t rb = (pb - split) * (int64_t)stride + head_off;
            const char* ca = make_uniform(reinterpret_cast<const char*>(p.cache) + ra);
            const char* cb = make_uniform(reinterpret_cast<const char*>(p.cache) + rb);
            const char* sa = make_uniform(reinterpret_cast<const char*>(p.scale) + (ra / kQuantGroup) * 2);
            const char* sb = make_uniform(reinterpret_cast<const char*>(p.scale) + (rb / kQuantGroup) * 2);
            dma_stage_paged(dst, ca, cb, sa, sb, split, off, kv_off, kv_off_s);
        } else {
            const char* cb = make_uniform(g.cbase + idx * step_c);
            const char* sb = make_uniform(reinterpret_cast<const char*>(p.scale) +
                                          ((g.cbase - reinterpret_cast<const char*>(p.cache)) / kQuantGroup) * 2 + idx * step_s);
            dma_stage(dst, cb, sb, off, kv_off, kv_off_s);
        }
    };
    auto issue = [&](const Segment& g, int idx, int slot) {
        if (idx == g.n_stages - 1 && g.tail_rows_mem < kStageTokens) { // wave-uniform, at most once per segment
            // When the last row is the new token, which this wave has yet to write, the overhanging rows are clamped
            // onto the token before it instead: they are masked, but their V scales are multiplied by zero
            // probabilities and have to be finite, which the bytes of a row nobody has written need not be.
            const int rows_mem = g.tail_rows_mem - ((g.has_new && g.tail_rows_mem >= 2) ? 1 : 0);
            DmaOffsets tail;
            make_dma_offsets(tail, lane, stride, sstride_b, rows_mem);
            issue_with(g, idx, slot, tail, rows_mem);
        } else {
            issue_with(g, idx, slot, full, kStageTokens);
        }
    };

    // Virtual heads (sub_shift > 0): which part of the 128 channels is the column's head's, and which the lane holds
    const int row_len = kDh >> p.sub_shift; // head_dim: channels of a row of the query / output tensors
    const int chan_off = (32 * kq) & (row_len - 1); // the lane's 32 channels inside such a row
    // the lane's channels belong to the head in column m (columns past rep copy column 0)
    const bool q_keep = ((32 * kq) >> (7 - p.sub_shift)) == ((m < p.rep ? m : 0) / (p.rep >> p.sub_shift));
    auto keep_own_channels = [&](half8_t (&q)[2][2]) { // (after the query loads have landed)
        if (!q_keep) {
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int e = 0; e < 8; ++e) q[jj][i][e] = (half_t)0.f;
        }
    };
    // Q^T as the B operand, kept for a whole segment: q[j][i] = Q[head m][32*kq + 16*j + 8*i .. +7]
    // four query pieces (+ the lane's group of the sequence's new token)
    constexpr int kQueryLoads = 5;
    (void)kQueryLoads; // only the counted waits name it
    // lanes 0..15: groups of the new token's K row (this kv head), lanes 16..31: of its V row (upper half-wave mirrors)
    // untracked: by load16_untracked, for the hand-over inside a range (the caller waits); otherwise by ordinary
    // loads that are waited for on the spot (first segment of a range, token-split workgroups)
    auto load_query = [&](const Segment& g, half8_t (&q)[2][2], u32x4_t& newtok, auto untracked) {
        {
            const half_t* src = ((lane & 16) ? p.cur_value : p.cur_key) +
                                ((int64_t)g.qrow * p.kv_heads + kvh) * kDh + 8 * (lane & 15);
            if (untracked) load16_untracked(newtok, src);
            else newtok = *reinterpret_cast<const u32x4_t*>(src);
        }
        // Columns m >= rep of the MFMA have no query head: they carry a copy of head 0 of the group, whose results
        // are never stored.
        // (a row of the query tensor holds head_dim = row_len channels; the lane's 32 channels of the 128-channel
        // operand are channels chan_off .. + 31 of that row when they belong to the column's head, see q_keep)
        const half_t* qp =
            p.q + (((int64_t)g.qrow * p.num_heads) + (int64_t)kvh * p.rep + (m < p.rep ? m : 0)) * row_len + chan_off;
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                if (untracked) load16_untracked(q[jj][i], qp + 16 * jj + 8 * i);
                else q[jj][i] = *reinterpret_cast<const half8_t*>(qp + 16 * jj + 8 * i);
            }
        if (!untracked) { // the wait for these loads happens HERE, not in front of every stage's first MFMA
            asm volatile("" : "+v"(q[0][0]), "+v"(q[0][1]), "+v"(q[1][0]), "+v"(q[1][1]), "+v"(newtok));
            keep_own_channels(q);
        }
    };

    // When every wave owns a whole kv head (no token split inside the workgroup) nothing is combined through LDS, the
    // stage buffers stay private to their wave, and the first stage of the NEXT segment is put in flight before the
    // current segment's results are normalised and stored: the transition between two sequences costs no DMA bubble.
    constexpr bool direct = DIRECT;
    // When the waves of a workgroup share one kv head (token split) the transfers run TWO stages ahead: a stage is
    // read into registers at the top of its arithmetic, so its buffer can take the stage after next while the
    // arithmetic runs (measured: 8 x 32k..128k tokens on one kv head 55.2 -> 52.4 us; with a kv head per wave the
    // deeper queue is slower, 148 -> 160 us on 64 x 32 kv heads, so those keep one stage ahead).
    constexpr bool deep = !DIRECT;
    Segment cur, nxt;
    next_segment(cur);
    int slot0 = 0; // stage buffer of the current segment's stage 0
    // stage 0 of `cur` is already enqueued: by the previous segment's last stage, or here, AHEAD of the query loads,
    // whose wait (in load_query) would otherwise pass before the first transfer is even requested
    bool cur_in_flight = cur.n_stages > 0;
    if (cur_in_flight) issue(cur, 0, 0);
    // store instructions issued behind the stage-0 transfers of a segment that was put in flight early (see the waits)
    int pending_stores = 0;
    half8_t qB[2][2];
    u32x4_t newB = {0, 0, 0, 0};
    load_query(cur, qB, newB, std::false_type{});
    for (;;) {
        SoftmaxState ss;
#pragma unroll
        for (int i = 0; i < 8; ++i) ss.oacc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
        ss.m_run = -INFINITY;
        ss.l_part = 0.f;

        bool has_next = false;
        half8_t qN[2][2];
        u32x4_t newN = {0, 0, 0, 0};
        if (cur.n_stages > 0) {
            if (!cur_in_flight) issue(cur, 0, slot0);
            const int last = cur.n_stages - 1;
            // ---- every stage but the last. The buffer the next stage lands in was last read by the stage before this
            // one, which has finished in program order.
            for (int it = 0; it < last; ++it) {
                const int slot = (slot0 + it) & 1;
                if (!deep || it == 0) issue(cur, it + 1, slot ^ 1);
                // everything older than the transfers just enqueued has landed: stage `it`. The previous segment's
                // result stores were issued AFTER this segment's stage 0 (which was put in flight ahead of them), so
                // they may stay in flight: waiting for their acknowledgement here cost 2 us per sequence boundary.
                PPLHIP_WAIT_VMCNT_PLUS(kDmaPerStage, pending_stores);
                pending_stores = 0;
                __builtin_amdgcn_sched_barrier(0);
                compute_stage(wave_lds_addr + slot * kStageBytes, ro, ss, qB, kq, kStageTokens, p.score_scale, [&]() {
                    if (deep && it + 2 < cur.n_stages) issue(cur, it + 2, slot);
                });
                __builtin_amdgcn_sched_barrier(0);
            }
            // ---- the last stage, outside the loop: the next segment's queries are loaded around it, and what the
            // compiler knows about loads in flight must not travel around the loop above
            {
                const int slot = (slot0 + last) & 1;
                has_next = direct && pos < r1;
                if (has_next) {
                    next_segment(nxt);
                    load_query(nxt, qN, newN, std::true_type{}); // older than the transfers below
                    issue(nxt, 0, slot ^ 1);
                    PPLHIP_WAIT_VMCNT_PLUS(kDmaPerStage + kQueryLoads, pending_stores); // the last stage only
                } else {
                    PPLHIP_WAIT_VMCNT_PLUS(0, pending_stores);
                }
                pending_stores = 0;
                __builtin_amdgcn_sched_barrier(0);
                if (cur.has_new) {
                    // The stage has landed with whatever the slab held in the new token's row: the row is replaced in
                    // the stage buffer by the freshly quantised token (LDS operations of one wave execute in order, so
                    // the reads below see it), and the same bytes go to the slab.
                    if (lane < 32) {
                        const int grp = lane & 15, isv = lane >> 4, r = cur.tail_rows_valid - 1;
                        uint2 qv;
                        half_t sc;
                        quantize_group8(make_uint4(newB[0], newB[1], newB[2], newB[3]), &qv, &sc);
                        const uint32_t st = wave_lds_addr + slot * kStageBytes;
                        uint16_t sbits;
                        __builtin_memcpy(&sbits, &sc, 2);
                        lds_write_b64(st + (isv ? kLdsV : kLdsK) + r * 128 + (((grp >> 1) ^ (r & 7)) * 16) + (grp & 1) * 8,
                                      qv);
                        lds_write_b16(st + (isv ? kLdsVs : kLdsKs) + r * 32 + grp * 2, sbits);
                        if (cur.tail_rows_mem == 1) // the new token is the stage's only row: every row is a copy of it
                            for (int r2 = 1; r2 < kStageTokens; ++r2)
                                lds_write_b16(st + (isv ? kLdsVs : kLdsKs) + r2 * 32 + grp * 2, sbits);
                        // the token's K row of this kv head in the slab: r rows into the wave's last stage
                        const int64_t tl = (int64_t)(cur.n_stages - 1) * kStageTokens + r; // relative to t_begin
                        int64_t row;
                        if (PAGED) {
                            const int64_t ta = (int64_t)cur.t_begin + tl;
                            row = (cur.page_row[ta >> p.page_shift] + (ta & ((int64_t(1) << p.page_shift) - 1))) *
                                      (int64_t)stride + head_off;
                        } else {
                            row = (cur.cbase - reinterpret_cast<const char*>(p.cache)) + tl * (int64_t)stride;
                        }
                        row += isv ? kv_off : 0;
                        // (two more stores behind the next stage 0; the waits count only the result rows. A store in
                        // the middle of a wave's stream costs it about a stage: where the launch has write-only
                        // workgroups anyway, they take these rows.)
                        if (!p.new_tokens_written_elsewhere) {
                            *reinterpret_cast<uint2*>(p.cache + row + grp * 8) = qv;
                            p.scale[row / kQuantGroup + grp] = sc;
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                compute_stage(wave_lds_addr + slot * kStageBytes, ro, ss, qB, kq, cur.tail_rows_valid, p.score_scale,
                              []() {});
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        const float l_tot = wave_sum_over_quads(ss.l_part);

        if (direct) {
            // ---- straight from registers: lane (m, kq) holds channels 8*(4*kq + e) .. +7 of query head m in oacc[.][e]
            if (m < p.rep) {
                const int head = kvh * p.rep + m;
                if (cur.whole_sequence) {
                    // (virtual heads: only the head's own channels are output; every lane group issues its stores
                    // or none, the count behind the next stage 0 stays a lower bound)
                    half_t* dst = p.out + ((int64_t)cur.qrow * p.num_heads + head) * row_len + chan_off;
                    const float inv_l = 1.0f / l_tot;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        half_t o[8];
#pragma unroll
                        for (int i = 0; i < 8; ++i) o[i] = (half_t)(ss.oacc[i][e] * inv_l);
                        uint4 packed;
                        __builtin_memcpy(&packed, o, 16);
                        if (q_keep) *reinterpret_cast<uint4*>(dst + 8 * e) = packed;
                    }
                } else {
                    const int64_t prow = (s_idx + cur.b) * p.num_heads + head;
                    float* dst = p.part_acc + prow * kDh + 32 * kq;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        *reinterpret_cast<float4_t*>(dst + 8 * e) =
                            float4_t{ss.oacc[0][e], ss.oacc[1][e], ss.oacc[2][e], ss.oacc[3][e]};
                        *reinterpret_cast<float4_t*>(dst + 8 * e + 4) =
                            float4_t{ss.oacc[4][e], ss.oacc[5][e], ss.oacc[6][e], ss.oacc[7][e]};
                    }
                    if (kq == 0) {
                        p.part_ml[prow * 2 + 0] = ss.m_run;
                        p.part_ml[prow * 2 + 1] = l_tot;
                    }
                }
            }
        } else {
            // ---- combine the token splits of each kv head: LDS layout [wave][head][Dh + 2] (acc, then max, sum),
            // reusing the stage buffers
            __syncthreads();
            if (m < p.rep) {
                float* dst = lds + ((size_t)wave * p.rep + m) * row_f;
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int i = 0; i < 8; ++i) dst[8 * (4 * kq + e) + i] = ss.oacc[i][e];
                if (kq == 0) {
                    dst[kDh] = ss.m_run;
                    dst[kDh + 1] = l_tot;
                }
            }
            __syncthreads();
            const int n_out = p.hpb * p.rep * kDh; // (kv head of the group, query head of the kv head, channel)
            for (int idx = threadIdx.x; idx < n_out; idx += kDecodeWaves * kWave) {
                const int d = idx & (kDh - 1);
                const int hh = idx >> 7; // kv_local * rep + h
                const int kl = hh / p.rep, h = hh - kl * p.rep;
                float mx = -INFINITY;
                for (int t = 0; t < tsplits; ++t)
                    mx = fmaxf(mx, lds[((size_t)(t * p.hpb + kl) * p.rep + h) * row_f + kDh]);
                float acc = 0.f, l = 0.f;
                for (int t = 0; t < tsplits; ++t) {
                    const float* src = lds + ((size_t)(t * p.hpb + kl) * p.rep + h) * row_f;
                    const float wgt = __builtin_amdgcn_exp2f(src[kDh] - mx); // a wave without tokens: max -inf -> 0
                    acc += wgt * src[d];
                    l += wgt * src[kDh + 1];
                }
                const int head = (hg * p.hpb + kl) * p.rep + h;
                if (cur.whole_sequence) {
                    if ((d >> (7 - p.sub_shift)) == h / (p.rep >> p.sub_shift)) // (virtual heads: the head's own channels)
                        p.out[((int64_t)cur.qrow * p.num_heads + head) * row_len + (d & (row_len - 1))] = (half_t)(acc / l);
                } else {
                    const int64_t prow = (s_idx + cur.b) * p.num_heads + head;
                    p.part_acc[prow * kDh + d] = acc;
                    if (d == 0) {
                        p.part_ml[prow * 2 + 0] = mx;
                        p.part_ml[prow * 2 + 1] = l;
                    }
                }
            }
            __syncthreads(); // the next segment's transfers overwrite the combine area
        }

        if (has_next) { // its stage 0 is already in flight, in the buffer the last stage did not use
            // (has_next implies the register epilogue: 4 16-byte stores of a finished row, or 8 of a partial result.
            // The count is a lower bound on the store instructions behind the next segment's stage 0 -- the small
            // ones, which the compiler may merge, are left out -- so a wait that allows this many more operations in
            // flight still covers stage 0 and everything older.)
            pending_stores = cur.whole_sequence ? 4 : 8;
            // the next segment's queries (and new token) are older than its stage 0: landed after this wait
            PPLHIP_WAIT_VMCNT_PLUS(kDmaPerStage, pending_stores);
            slot0 = (slot0 + cur.n_stages) & 1;
            cur = nxt;
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                for (int i = 0; i < 2; ++i) qB[jj][i] = qN[jj][i];
            keep_own_channels(qB);
            newB = newN;
            cur_in_flight = true;
        } else {
            if (pos >= r1) break;
            next_segment(cur);
            slot0 = 0;
            cur_in_flight = cur.n_stages > 0;
            if (cur_in_flight) issue(cur, 0, 0);
            load_query(cur, qB, newB, std::false_type{});
        }
    }
}

template <bool PAGED, bool DIRECT>
__global__ __launch_bounds__(kDecodeWaves* kWave, 2) void decode_int8kv_kernel(const DecodeParams p) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    decode_workgroup<PAGED, DIRECT>(p, blockIdx.x, smem);
}

// One workgroup per (decode sequence, query head): kMergeGroups groups of 32 lanes stride over the partial slots of the
// sequence (one per range it touches), each lane owning 4 channels; the groups' running (max, sum, acc) are combined
// through LDS. Every step of a group is a memory round trip for four slots, so the group count follows the slots per
// sequence: sixteen where sequences span dozens of ranges (63 slots: one round trip), four where they span a few (half
// the waves to launch: 5.8 -> 4.8 us on 120 sequences over 256 ranges).
// out[d] = sum_s w_s acc_s[d] / sum_s w_s l_s with w_s = exp2(m_s - max_s m_s). Sequences that lie inside a single
// range were already written by the decode kernel.
template <int kMergeGroups, int kSlotsPerStep>
__global__ __launch_bounds__(32 * kMergeGroups) void decode_merge_kernel(const DecodeParams p) {
    __shared__ float red[kMergeGroups][kDh + 2];
    const int head = blockIdx.x;
    const int g = threadIdx.x >> 5;
    const int d4 = (threadIdx.x & 31) * 4;
    const int64_t total = p.kvstarts[p.nd] + (int64_t)p.nd * kBoundaryTokens; // virtual positions, as in the decode kernel
    const int64_t R = range_tokens(total, p.num_ranges);
    // blockIdx.y is a sequence, or (when there are more sequences than ranges) a boundary between two ranges: only
    // a sequence that straddles a boundary has anything to merge, and it is handled by the first boundary it crosses
    int b;
    if (p.merge_by_boundary) {
        const int64_t edge = ((int64_t)blockIdx.y + 1) * R; // first token of range blockIdx.y + 1
        if (edge >= total) return;
        b = p.range_first[blockIdx.y + 1]; // the sequence that holds position `edge` (found by the decode kernel)
        const int64_t vb = p.kvstarts[b] + (int64_t)b * kBoundaryTokens;
        if (vb >= edge || div_positions(vb, R) != blockIdx.y) return; // starts there, or crossed a boundary before this one
    } else {
        b = blockIdx.y;
    }
    const int64_t vlo = p.kvstarts[b] + (int64_t)b * kBoundaryTokens;
    const int64_t s_lo = div_positions(vlo, R), s_hi = div_positions(vlo + (p.kvstarts[b + 1] - p.kvstarts[b]) - 1, R);
    if (s_lo == s_hi) return;
    float mx = -INFINITY, l = 0.f;
    float4_t acc = {0.f, 0.f, 0.f, 0.f};
    // kSlotsPerStep slots per step, their loads issued together: a long sequence has dozens of slots per lane group,
    // and one memory latency per slot would add up. A step that runs past the sequence's last slot re-reads that slot
    // and gives it no weight, so that every step is the same loads (a remainder walked one slot at a time cost some
    // lane groups three more round trips on sequences of 63 slots). Where sequences have a handful of slots a lane
    // group gets one or two of them and takes them one at a time.
    for (int64_t s = s_lo + g; s <= s_hi; s += kSlotsPerStep * kMergeGroups) {
        float mc[kSlotsPerStep], lc[kSlotsPerStep];
        float4_t a[kSlotsPerStep];
#pragma unroll
        for (int u = 0; u < kSlotsPerStep; ++u) {
            const int64_t su = s + u * kMergeGroups;
            const int64_t prow = ((su <= s_hi ? su : s_hi) + b) * p.num_heads + head;
            mc[u] = p.part_ml[prow * 2];
            lc[u] = p.part_ml[prow * 2 + 1];
            a[u] = *reinterpret_cast<const float4_t*>(p.part_acc + prow * kDh + d4);
            if (su > s_hi) mc[u] = -INFINITY;
        }
#pragma unroll
        for (int u = 0; u < kSlotsPerStep; ++u) {
            const float m_new = fmaxf(mx, mc[u]);
            // (the first slot of a lane group is always a real one, so m_new is finite from there on)
            const float w_old = __builtin_amdgcn_exp2f(mx - m_new), w_new = __builtin_amdgcn_exp2f(mc[u] - m_new);
            acc = acc * w_old + a[u] * w_new;
            l = l * w_old + lc[u] * w_new;
            mx = m_new;
        }
    }
    red[g][d4 + 0] = acc[0];
    red[g][d4 + 1] = acc[1];
    red[g][d4 + 2] = acc[2];
    red[g][d4 + 3] = acc[3];
    if ((threadIdx.x & 31) == 0) {
        red[g][kDh] = mx;
        red[g][kDh + 1] = l;
    }
    __syncthreads();
    if (threadIdx.x < kDh) {
        const int d = threadIdx.x;
        float M = -INFINITY;
#pragma unroll
        for (int i = 0; i < kMergeGroups; ++i) M = fmaxf(M, red[i][kDh]);
        float a = 0.f, L = 0.f;
#pragma unroll
        for (int i = 0; i < kMergeGroups; ++i) {
            const float w = __builtin_amdgcn_exp2f(red[i][kDh] - M); // groups that saw no slot have max -inf -> 0
            a += w * red[i][d];
            L += w * red[i][kDh + 1];
        }
        // (virtual heads, see DecodeParams::sub_shift: only the head's own channels are output)
        const int row_len = kDh >> p.sub_shift;
        if ((d >> (7 - p.sub_shift)) == (head % p.rep) / (p.rep >> p.sub_shift))
            p.out[(p.seqstarts[b] * p.num_heads + head) * row_len + (d & (row_len - 1))] = (half_t)(a / L);
    }
}

int decode_blocks_per_cu() {
    return (160 * 1024) / kDecodeLdsBytes; // LDS-limited
}

int decode_waves_per_block() {
    return kDecodeWaves;
}

// Head dims 64 and 32 run the decode kernel with 2 (4) neighbouring kv heads as one head of 128 channels when the
// heads are neighbours in the slab, their number divides, and the query heads of such a group fit the 16 columns.
// (The number of kv heads the kernel then sees: num_kv_heads >> shift; 0 = not this way.)
int decode_virtual_heads(const pplhip_mhca_args* a) {
    const int shift = a->head_dim == 64 ? 1 : a->head_dim == 32 ? 2 : -1;
    if (shift < 0 || a->d_attn_mask != nullptr || a->num_kv_heads <= 0) return 0;
    if (a->num_kv_heads % (1 << shift) || a->cache_stride_h != a->head_dim) return 0;
    if (a->num_heads % a->num_kv_heads || ((a->num_heads / a->num_kv_heads) << shift) > 16) return 0;
    return a->num_kv_heads >> shift;
}

int decode_heads_per_block(int kv_heads) {
    int hpb = 1;
    while (hpb < kDecodeWaves && kv_heads % (hpb * 2) == 0) hpb *= 2;
    return hpb;
}

// More than 64 KiB of dynamic LDS per workgroup needs an explicit opt-in per kernel, once per device (the attribute is
// kept per device by the runtime); setting it twice from two threads is harmless, so a relaxed bit mask is enough.
static pplhip_retcode reserve_decode_lds(std::atomic<uint64_t>& done, std::initializer_list<const void*> kernels) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        PPLHIP_FAIL(PPLHIP_RC_DEVICE_RUNTIME_ERROR, "decode: no current device");
    if (done.load(std::memory_order_relaxed) >> dev & 1) return PPLHIP_RC_SUCCESS;
    for (const void* fn : kernels) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kDecodeLdsBytes);
        if (e != hipSuccess)
            PPLHIP_FAIL(PPLHIP_RC_DEVICE_RUNTIME_ERROR, "decode: cannot reserve %d bytes of LDS per workgroup: %s",
                        kDecodeLdsBytes, hipGetErrorString(e));
    }
    done.fetch_or(uint64_t(1) << dev, std::memory_order_relaxed);
    return PPLHIP_RC_SUCCESS;
}

// Fills the launch parameters of the decode sequences' attention; *blocks: workgroups of the launch.
// a->head_dim 128, or 64 / 32 where decode_virtual_heads() allows it.
static pplhip_retcode decode_setup(const pplhip_mhca_args* a, const pplhip_mhca_plan* plan, void* ws, DecodeParams* out,
                                   int64_t* out_blocks) {
    const int nd = (int)a->decoding_batches;
    const int sub_shift = a->head_dim == 128 ? 0 : a->head_dim == 64 ? 1 : 2;
    if (a->head_dim != (kDh >> sub_shift) || (sub_shift && !decode_virtual_heads(a)))
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "decode: head_dim %d does not run this kernel", a->head_dim);
    DecodeParams p;
    p.q = (const half_t*)a->d_query;
    p.cur_key = (const half_t*)a->d_current_key;
    p.cur_value = (const half_t*)a->d_current_value;
    p.cache = (int8_t*)a->d_cache;
    p.scale = (half_t*)a->d_scale;
    p.seqstarts = a->d_seqstarts;
    p.kvstarts = a->d_kvstarts;
    p.cachestarts = a->d_cachestarts;
    p.cs_stride_b = a->cachestart_stride_b;
    p.page_shift = page_shift_of(a->cache_mode, a->page_size);
    p.out = (half_t*)a->d_output;
    p.addr = CacheAddr{a->cache_stride_s, a->cache_stride_l, a->cache_stride_h << sub_shift, a->cache_stride_kv,
                       a->layer_idx};
    p.nd = nd;
    p.num_heads = a->num_heads;
    p.kv_heads = a->num_kv_heads >> sub_shift;
    p.rep = (a->num_heads / a->num_kv_heads) << sub_shift;
    p.sub_shift = sub_shift;
    p.num_ranges = plan->decode_num_ranges;
    p.hpb = decode_heads_per_block(p.kv_heads);
    p.score_scale = 1.4426950408889634f / sqrtf((float)a->head_dim);
    if (p.num_ranges <= 0 || plan->decode_heads_per_block != p.hpb)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "decode: plan was not produced by pplhip_mhca_prepare for these arguments");
    if (ws == nullptr) PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "decode: needs the workspace reported by pplhip_mhca_prepare");
    const size_t slots = (size_t)p.num_ranges + nd;
    p.part_acc = (float*)ws;
    p.part_ml = (float*)((char*)ws + slots * p.num_heads * kDh * sizeof(float));
    p.range_first = (int32_t*)((char*)ws + slots * p.num_heads * (kDh + 2) * sizeof(float));
    const int64_t blocks = (int64_t)p.num_ranges * (p.kv_heads / p.hpb);
    if (blocks > 0x7fffffffLL) PPLHIP_FAIL(PPLHIP_RC_OUT_OF_RANGE, "decode: too many tasks");
    p.merge_by_boundary = nd > p.num_ranges - 1;
    p.new_tokens_written_elsewhere = 0;
    *out = p;
    *out_blocks = blocks;
    return PPLHIP_RC_SUCCESS;
}

// the sequences that need merging are those that straddle a range boundary: at most num_ranges - 1 of them, however
// many sequences there are (2048 short sequences launched 65k workgroups that all left at once: 35 us)
static pplhip_retcode launch_decode_merge(const DecodeParams& p, hipStream_t stream) {
    const dim3 grid(p.num_heads, p.merge_by_boundary ? p.num_ranges - 1 : p.nd);
    // lane groups per workgroup by the slots a sequence has on average (ranges / sequences + 1): with dozens of slots
    // every group takes four per memory round trip, with a handful one
    if (p.num_ranges >= 32 * p.nd)
        hipLaunchKernelGGL((decode_merge_kernel<16, 4>), grid, dim3(512), 0, stream, p);
    else if (p.num_ranges >= 16 * p.nd)
        hipLaunchKernelGGL((decode_merge_kernel<8, 4>), grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL((decode_merge_kernel<4, 1>), grid, dim3(128), 0, stream, p);
    PPLHIP_CHECK_LAUNCH("decode_merge");
    return PPLHIP_RC_SUCCESS;
}

pplhip_retcode launch_decode(const pplhip_mhca_args* a, const pplhip_mhca_plan* plan, void* ws, hipStream_t stream,
                             bool new_tokens_in_slab) {
    if (a->decoding_batches == 0) return PPLHIP_RC_SUCCESS;
    DecodeParams p;
    int64_t blocks;
    pplhip_retcode rc = decode_setup(a, plan, ws, &p, &blocks);
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    p.new_tokens_written_elsewhere = new_tokens_in_slab;
    const size_t lds_bytes = kDecodeLdsBytes; // stage buffers; the final combine (4 * rep * 130 floats) reuses them
    static std::atomic<uint64_t> lds_opted_in{0};
    rc = reserve_decode_lds(lds_opted_in, {reinterpret_cast<const void*>(decode_int8kv_kernel<false, false>),
                                           reinterpret_cast<const void*>(decode_int8kv_kernel<true, false>),
                                           reinterpret_cast<const void*>(decode_int8kv_kernel<false, true>),
                                           reinterpret_cast<const void*>(decode_int8kv_kernel<true, true>)});
    if (rc != PPLHIP_RC_SUCCESS) return rc;
    const dim3 grid((unsigned)blocks), block(kDecodeWaves * kWave);
    const bool direct = p.hpb == kDecodeWaves;
    if (p.page_shift && direct)
        hipLaunchKernelGGL((decode_int8kv_kernel<true, true>), grid, block, lds_bytes, stream, p);
    else if (p.page_shift)
        hipLaunchKernelGGL((decode_int8kv_kernel<true, false>), grid, block, lds_bytes, stream, p);
    else if (direct)
        hipLaunchKernelGGL((decode_int8kv_kernel<false, true>), grid, block, lds_bytes, stream, p);
    else
        hipLaunchKernelGGL((decode_int8kv_kernel<false, false>), grid, block, lds_bytes, stream, p);
    PPLHIP_CHECK_LAUNCH("decode_int8kv");
    return launch_decode_merge(p, stream);
}

} // namespace pplhip
