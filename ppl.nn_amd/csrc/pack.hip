// On-device rebuild of the ragged-batch tables (seqstarts / kvstarts / cachestarts / start_pos) from per-slot
// state: stable compaction with decode sequences first, then prefill sequences, then prefix sums and maxima.
// At most 1024 slots, so one workgroup does everything in LDS; the kernel is latency-bound (a few microseconds)
// and replaces eight host-to-device uploads per step.
#include "common.h"
#include "table_check.h"

namespace pplhip {

constexpr int kMaxSlots = 1024;

struct PackParams {
    int64_t* slot_kvlen; // written only when `advance` is set
    const int64_t* slot_newlen;
    const int64_t* slot_cachestart;
    int64_t* seqstarts;
    int64_t* kvstarts;
    int64_t* cachestarts;
    int64_t* start_pos;
    int64_t* batch_slots;
    int64_t* header;
    int32_t n;
    int32_t advance; // slot_kvlen += slot_newlen once the tables are built
};

// Inclusive scans and maxima across the workgroup: inside a wave with lane shuffles (six steps, no barrier), then one
// LDS entry per wave that every thread adds up for the waves in front of it. Two values travel together. (Scans of
// the whole workgroup through LDS, one barrier per doubling step, made this kernel 7.5 us of barriers.)
__device__ inline int64_t wave_inclusive_scan(int64_t v) {
    const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const int64_t x = __shfl_up(v, off);
        if (lane >= off) v += x;
    }
    return v;
}
__device__ inline int64_t wave_max(int64_t v) {
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const int64_t x = __shfl_xor(v, off);
        v = x > v ? x : v;
    }
    return v;
}
constexpr int kMaxWaves = kMaxSlots / kWave;
// a, b: this thread's values in, their inclusive sums over threads 0 .. tid out; per_wave: [2][kMaxWaves]
__device__ inline void block_inclusive_scan2(int64_t& a, int64_t& b, int64_t* per_wave) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    a = wave_inclusive_scan(a);
    b = wave_inclusive_scan(b);
    if (lane == kWave - 1) {
        per_wave[wave] = a;
        per_wave[kMaxWaves + wave] = b;
    }
    __syncthreads();
    int64_t pa = 0, pb = 0;
    for (int w = 0; w < wave; ++w) {
        pa += per_wave[w];
        pb += per_wave[kMaxWaves + w];
    }
    a += pa;
    b += pb;
    __syncthreads(); // (per_wave is used again)
}
// maxima of a and of b over the workgroup's threads
__device__ inline void block_max2(int64_t& a, int64_t& b, int64_t* per_wave, int nwaves) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    a = wave_max(a);
    b = wave_max(b);
    if (lane == 0) {
        per_wave[wave] = a;
        per_wave[kMaxWaves + wave] = b;
    }
    __syncthreads();
    for (int w = 0; w < nwaves; ++w) {
        a = per_wave[w] > a ? per_wave[w] : a;
        b = per_wave[kMaxWaves + w] > b ? per_wave[kMaxWaves + w] : b;
    }
    __syncthreads();
}

__global__ __launch_bounds__(kMaxSlots) void pack_tables_kernel(const PackParams p) {
    __shared__ int64_t per_wave[2 * kMaxWaves];
    __shared__ int64_t packed_new[kMaxSlots];
    __shared__ int64_t packed_kv[kMaxSlots];
    const int tid = threadIdx.x;
    const int nt = blockDim.x; // a multiple of 64
    const bool in = tid < p.n;
    const int64_t kl = in ? p.slot_kvlen[tid] : 0;
    const int64_t nl = in ? p.slot_newlen[tid] : 0;
    const bool active = nl > 0;
    const bool is_decode = active && nl == 1 && kl > 0;
    const bool is_prefill = active && !is_decode;

    int64_t dec_incl = is_decode ? 1 : 0, pre_incl = is_prefill ? 1 : 0;
    block_inclusive_scan2(dec_incl, pre_incl, per_wave);
    __shared__ int64_t totals[2];
    if (tid == nt - 1) {
        totals[0] = dec_incl;
        totals[1] = pre_incl;
    }
    packed_new[tid] = 0;
    packed_kv[tid] = 0;
    __syncthreads();
    const int64_t nd = totals[0];
    const int64_t batch = nd + totals[1];
    int64_t pos = -1;
    if (is_decode) pos = dec_incl - 1;
    if (is_prefill) pos = nd + pre_incl - 1;
    if (pos >= 0) {
        packed_new[pos] = nl;
        packed_kv[pos] = kl + nl;
        p.cachestarts[pos] = p.slot_cachestart[tid];
        p.start_pos[pos] = kl;
        p.batch_slots[pos] = tid;
    }
    __syncthreads();
    const int64_t my_new = packed_new[tid], my_kv = packed_kv[tid];
    int64_t seq_incl = my_new, kv_incl = my_kv;
    block_inclusive_scan2(seq_incl, kv_incl, per_wave);
    int64_t max_new = my_new, max_kv = my_kv;
    block_max2(max_new, max_kv, per_wave, nt / kWave);
    if (tid < p.n) {
        p.seqstarts[tid + 1] = seq_incl; // entries past the batch repeat the total (their packed lengths are 0)
        p.kvstarts[tid + 1] = kv_incl;
        if (tid >= batch) {
            p.cachestarts[tid] = 0;
            p.start_pos[tid] = 0;
            p.batch_slots[tid] = -1;
        }
    }
    if (tid == 0) {
        p.seqstarts[0] = 0;
        p.kvstarts[0] = 0;
    }
    // (every thread read its own slot's state at the top and nothing else reads it: the state may move on in place)
    if (p.advance && in && nl > 0) p.slot_kvlen[tid] = kl + nl;
    if (tid == nt - 1) {
        p.header[0] = batch;
        p.header[1] = nd;
        p.header[2] = max_new;
        p.header[3] = max_kv;
        p.header[4] = seq_incl;
        p.header[5] = kv_incl;
    }
}

pplhip_retcode launch_pack_tables(const pplhip_pack_args* a, hipStream_t stream) {
    if (a->num_slots <= 0 || a->num_slots > kMaxSlots)
        PPLHIP_FAIL(PPLHIP_RC_INVALID_VALUE, "pack_tables: num_slots %d outside [1, %d]", a->num_slots, kMaxSlots);
    PackParams p{const_cast<int64_t*>(a->d_slot_kvlen), a->d_slot_newlen, a->d_slot_cachestart, a->d_seqstarts,
                 a->d_kvstarts, a->d_cachestarts, a->d_start_pos, a->d_batch_slots, a->d_header, a->num_slots,
                 a->advance_slots != 0};
    int threads = 64;
    while (threads < a->num_slots) threads <<= 1;
    hipLaunchKernelGGL(pack_tables_kernel, dim3(1), dim3(threads), 0, stream, p);
    PPLHIP_CHECK_LAUNCH("pack_tables");
    return PPLHIP_RC_SUCCESS;
}

__global__ void advance_slots_kernel(int64_t* kvlen, const int64_t* newlen, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && newlen[i] > 0) kvlen[i] += newlen[i];
}

pplhip_retcode launch_advance_slots(int64_t* kvlen, const int64_t* newlen, int n, hipStream_t stream) {
    if (n <= 0) return PPLHIP_RC_SUCCESS;
    hipLaunchKernelGGL(advance_slots_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, kvlen, newlen, n);
    PPLHIP_CHECK_LAUNCH("advance_slots");
    return PPLHIP_RC_SUCCESS;
}

// ---------------------------------------------------------------------------------------------------------------
// Consistency check of one call's tables (a debugging aid: the attention kernels trust the tables, and one bad entry
// is an out-of-range slab access). Reads the tables only; never touches the slab. One workgroup walks the sequences;
// the lowest (sequence, code) pair found wins, so the report does not depend on thread timing.
__global__ __launch_bounds__(256) void check_tables_kernel(const TableView p, int32_t* flag) {
    __shared__ unsigned long long first_bad;
    if (threadIdx.x == 0) first_bad = check_table_ends(p);
    __syncthreads();
    for (int64_t b = threadIdx.x; b < p.batch; b += blockDim.x) {
        const int code = check_table_sequence(p, b);
        if (code != PPLHIP_TABLES_OK) atomicMin(&first_bad, (unsigned long long)table_finding(b, code));
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const bool bad = first_bad != kNoTableFinding;
        flag[0] = bad ? (int32_t)(first_bad & 0xff) : PPLHIP_TABLES_OK; // [0] = code, [1] = first offending sequence
        flag[1] = bad ? (int32_t)(first_bad >> 8) : -1;
    }
}

TableView table_view_of(const pplhip_mhca_args* a, int64_t max_slab_tokens) {
    return TableView{a->d_seqstarts, a->d_kvstarts, a->d_cachestarts, a->d_start_pos, a->batch, a->decoding_batches,
                     a->max_seqlen, a->max_kvlen, a->total_new_tokens, max_slab_tokens, a->cachestart_stride_b,
                     page_shift_of(a->cache_mode, a->page_size)};
}

pplhip_retcode launch_check_tables(const pplhip_mhca_args* a, int64_t max_slab_tokens, int32_t* d_flag,
                                   hipStream_t stream) {
    hipLaunchKernelGGL(check_tables_kernel, dim3(1), dim3(256), 0, stream, table_view_of(a, max_slab_tokens), d_flag);
    PPLHIP_CHECK_LAUNCH("check_tables");
    return PPLHIP_RC_SUCCESS;
}

// the same rules over tables that live in host memory
void check_tables_host(const pplhip_mhca_args* a, int64_t max_slab_tokens, int32_t* flag) {
    const TableView p = table_view_of(a, max_slab_tokens);
    uint64_t first_bad = check_table_ends(p);
    for (int64_t b = 0; b < p.batch; ++b) {
        const int code = check_table_sequence(p, b);
        if (code != PPLHIP_TABLES_OK && table_finding(b, code) < first_bad) first_bad = table_finding(b, code);
    }
    const bool bad = first_bad != kNoTableFinding;
    flag[0] = bad ? (int32_t)(first_bad & 0xff) : PPLHIP_TABLES_OK;
    flag[1] = bad ? (int32_t)(first_bad >> 8) : -1;
}

} // namespace pplhip
