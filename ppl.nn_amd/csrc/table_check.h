// Consistency rules of one call's ragged-batch tables, shared by the device kernel behind pplhip_check_tables and the
// host loop behind pplhip_check_tables_host (internal; the codes are the PPLHIP_TABLES_* of the C ABI header).
#ifndef PPLHIP_CSRC_TABLE_CHECK_H_
#define PPLHIP_CSRC_TABLE_CHECK_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ppl_llm_kernel_hip.h"

namespace pplhip {

struct TableView {
    const int64_t* seqstarts;
    const int64_t* kvstarts;
    const int64_t* cachestarts;
    const int64_t* start_pos;
    int64_t batch, nd, max_seqlen, max_kvlen, total_new_tokens, max_slab_tokens, cs_stride_b;
    int32_t page_shift; // 0: one contiguous slab region per sequence
};

// A finding is ordered by (sequence, code): the lowest one is what a check reports, on the host and on the device alike.
__host__ __device__ inline uint64_t table_finding(int64_t b, int code) {
    return ((uint64_t)b << 8) | (uint64_t)code;
}
constexpr uint64_t kNoTableFinding = ~0ull;

// what the table ends say (entries 0 and batch), or kNoTableFinding
__host__ __device__ inline uint64_t check_table_ends(const TableView& p) {
    if (p.batch <= 0) return kNoTableFinding;
    uint64_t f = kNoTableFinding;
    if (p.seqstarts[p.batch] != p.total_new_tokens) f = table_finding(p.batch - 1, PPLHIP_TABLES_BAD_SEQSTARTS);
    if (p.kvstarts[0] != 0) f = table_finding(0, PPLHIP_TABLES_BAD_KVSTARTS);
    if (p.seqstarts[0] != 0) f = table_finding(0, PPLHIP_TABLES_BAD_SEQSTARTS);
    return f;
}

// the lowest code sequence b violates, or PPLHIP_TABLES_OK. Reads the tables only.
__host__ __device__ inline int check_table_sequence(const TableView& p, int64_t b) {
    const int64_t s0 = p.seqstarts[b], seqlen = p.seqstarts[b + 1] - s0;
    const int64_t kvlen = p.kvstarts[b + 1] - p.kvstarts[b];
    const int64_t sp = p.start_pos[b];
    if (seqlen < 1) return PPLHIP_TABLES_BAD_SEQSTARTS;
    if (kvlen < seqlen) return PPLHIP_TABLES_BAD_KVSTARTS;
    if (sp < 0 || kvlen != sp + seqlen) return PPLHIP_TABLES_KVLEN_MISMATCH;
    if (b < p.nd && (seqlen != 1 || s0 != b)) return PPLHIP_TABLES_BAD_DECODE_ORDER;
    if (seqlen > p.max_seqlen || kvlen > p.max_kvlen) return PPLHIP_TABLES_MAX_EXCEEDED;
    if (p.page_shift == 0) {
        const int64_t cs = p.cachestarts[b];
        return (cs < 0 || cs > p.max_slab_tokens - kvlen) ? PPLHIP_TABLES_SLAB_RANGE : PPLHIP_TABLES_OK;
    }
    const int64_t page = int64_t(1) << p.page_shift;
    const int64_t pages = (kvlen + page - 1) >> p.page_shift;
    if (pages > p.cs_stride_b) return PPLHIP_TABLES_PAGE_TABLE_TOO_SHORT;
    for (int64_t pg = 0; pg < pages; ++pg) {
        const int64_t first = p.cachestarts[b * p.cs_stride_b + pg];
        const int64_t left = kvlen - (pg << p.page_shift);
        const int64_t used = left < page ? left : page;
        if (first < 0 || first > p.max_slab_tokens - used) return PPLHIP_TABLES_SLAB_RANGE;
    }
    return PPLHIP_TABLES_OK;
}

} // namespace pplhip

#endif
