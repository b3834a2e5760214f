// Addressing of a latent cache shared by the sparse-MLA kernels: contiguous per request, one pool of
// rows, or a pool of pages behind a block table.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace mla {

// Where the rows of a request live. Without a block table a request's rows are
// kv + (b * batch_rows + key) * row bytes (batch_rows == 0: one pool shared by all requests,
// keys are pool rows). With a block table keys are logical positions of the request and
// logical page p = key >> page_shift lives at physical page block_table[b * table_stride + p].
struct KvAddressing {
    const int* block_table;
    int table_stride;
    int page_shift;
    int batch_rows;
};

// selected key -> row of the cache block, or -1 for padding (negative keys, keys beyond the
// block table, unmapped pages, rows beyond the cache)
__device__ __forceinline__ int resolve_key(int key, int b, const KvAddressing& kva, int n_kv_rows) {
    if (kva.block_table != nullptr) {
        const int page_no = key >> kva.page_shift;
        if (key < 0 || page_no >= kva.table_stride) return -1;
        const int page = kva.block_table[(size_t)b * kva.table_stride + page_no];
        if (page < 0) return -1;
        const long long row =
            ((long long)page << kva.page_shift) + (key & ((1 << kva.page_shift) - 1));
        return row < n_kv_rows ? (int)row : -1;
    }
    return key >= 0 && key < n_kv_rows ? key : -1;
}

}  // namespace mla
