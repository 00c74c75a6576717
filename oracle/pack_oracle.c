/* CPU oracle for the communicator buffer layout.  TEST INFRASTRUCTURE ONLY.
 *
 * A sequential restatement of the two CUDA kernels the reference embeds as
 * strings in chainerkfac/communicators/pure_nccl_communicator.py:
 *   cupy_batched_pack_arrays    (:300-377)
 *   cupy_batched_unpack_arrays  (:380-463)
 * Each "thread" of the original becomes one iteration of the tid loop; the
 * binary search over the cumulative size table, the row/column split, the
 * r(r+1)/2 + c slot formula, the rank filter and the division by `divisor`
 * are kept as written there.  Only the float32 <-> float32 cast pair is
 * restated (the reference hard-wires its communication dtype to float32,
 * pure_nccl_communicator.py:32-33).
 *
 * Pinned by tests/test_oracle_pack.py against numpy.tril_indices and a
 * pure-Python brute force.  Built by __graft_entry__.build() into
 * oracle/libpack_oracle.so; used by tests and by bench.py's cpu_baseline.
 */
#include <stdint.h>
#include <stddef.h>

static int find_array(const int *size_csum, int n_arrays, int tid)
{
    int j_min = 0;
    int j_max = n_arrays - 1;
    int j;
    for (;;) {
        j = (j_min + j_max) / 2;
        if (tid < size_csum[j]) {
            j_max = j - 1;
            continue;
        }
        if (tid >= size_csum[j + 1]) {
            j_min = j + 1;
            continue;
        }
        break;
    }
    return j;
}

/* pure_nccl_communicator.py:300-377 */
void oracle_pack_f32(float *dst_head, const int *dst_size_csum,
                     const uint64_t *list_src_dptr, const int *src_size_csum,
                     const int *triangle_size, const int *list_rank, int rank,
                     int total_threads, int n_arrays)
{
    for (int tid = 0; tid < total_threads; ++tid) {
        int j = find_array(src_size_csum, n_arrays, tid);
        if (rank >= 0 && list_rank[j] != rank) continue;
        const float *src = (const float *)(uintptr_t)list_src_dptr[j];
        int src_idx = tid - src_size_csum[j];
        int dst_idx;
        int matrix_size = triangle_size[j];
        if (matrix_size > 0) {
            int row_idx = src_idx / matrix_size;
            int col_idx = src_idx % matrix_size;
            if (col_idx > row_idx) continue;
            dst_idx = (row_idx * (row_idx + 1) / 2) + col_idx;
        } else {
            dst_idx = src_idx;
        }
        float *dst = dst_head + dst_size_csum[j];
        dst[dst_idx] = src[src_idx];
    }
}

/* pure_nccl_communicator.py:380-463 */
void oracle_unpack_f32(const uint64_t *list_dst_dptr, const int *dst_size_csum,
                       const float *src_head, const int *src_size_csum,
                       const int *triangle_size, const int *list_rank, int rank,
                       int divisor, int total_threads, int n_arrays)
{
    for (int tid = 0; tid < total_threads; ++tid) {
        int j = find_array(dst_size_csum, n_arrays, tid);
        if (rank >= 0 && list_rank[j] != rank) continue;
        float *dst = (float *)(uintptr_t)list_dst_dptr[j];
        int dst_idx = tid - dst_size_csum[j];
        int src_idx;
        int matrix_size = triangle_size[j];
        if (matrix_size > 0) {
            int row_idx = dst_idx / matrix_size;
            int col_idx = dst_idx % matrix_size;
            if (row_idx >= col_idx)
                src_idx = (row_idx * (row_idx + 1) / 2) + col_idx;
            else
                src_idx = (col_idx * (col_idx + 1) / 2) + row_idx;
        } else {
            src_idx = dst_idx;
        }
        const float *src = src_head + src_size_csum[j];
        float src_val = src[src_idx] / (float)divisor;
        dst[dst_idx] = src_val;
    }
}
