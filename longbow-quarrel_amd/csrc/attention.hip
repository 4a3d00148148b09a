// lq_attention: causal grouped-query attention over the paged cache, dispatch.
#include "common.h"

int lq_attention_generic(const void* q, int ldq, void* out, int ldo, int dtype, int rows, int nh,
                         int nkv, int hd, const int* row_pos, const int* row_seq,
                         const int* seq_slot, const int* block_table, int bt_stride,
                         const void* kcache, const void* vcache, int block_size, float scale,
                         int window, hipStream_t stream);

extern "C" int lq_attention(const void* q, int ldq, void* out, int ldo, int dtype, int rows, int nh,
                            int nkv, int hd, const int* row_pos, const int* row_seq,
                            const int* seq_slot, const int* block_table, int bt_stride,
                            const void* kcache, const void* vcache, int block_size, float scale,
                            int window, int force_generic, hipStream_t stream) {
  LQ_REQUIRE(rows > 0, "attention: rows %d must be positive", rows);
  LQ_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0, "attention: %d heads over %d kv heads", nh, nkv);
  LQ_REQUIRE(hd > 0 && block_size > 0 && bt_stride > 0, "attention: bad sizes");
  LQ_REQUIRE(ldq >= nh * hd && ldo >= nh * hd, "attention: a row stride is smaller than its row");
  LQ_REQUIRE(window >= 0, "attention: window %d must not be negative", window);
  (void)force_generic;
  return lq_attention_generic(q, ldq, out, ldo, dtype, rows, nh, nkv, hd, row_pos, row_seq,
                              seq_slot, block_table, bt_stride, kcache, vcache, block_size, scale,
                              window, stream);
}
