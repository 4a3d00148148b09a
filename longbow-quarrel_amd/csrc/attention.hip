// lq_attention: causal grouped-query attention over the paged cache, dispatch.
#include "common.h"

int lq_attention_generic(const void* q, int ldq, void* out, int ldo, int dtype, int rows, int batch, int nh,
                         int nkv, int hd, const int* row_pos, const int* row_seq,
                         const int* seq_slot, const int* block_table, int bt_stride,
                         const void* kcache, const void* vcache, int block_size, float scale,
                         int window, hipStream_t stream);
bool lq_attention_mfma_accepts(int dtype, int nh, int nkv, int hd, int block_size, int ldq, int ldo,
                               const void* q, const void* out, int decode);
long long lq_attention_mfma_workspace(int rows, int nh, int nkv, int hd, int max_len);
int lq_attention_mfma_unit_search(const int* pos, int rows, int nkv, int max_len);
int lq_attention_mfma(const void* q, int ldq, void* out, int ldo, int rows, int batch, int nh, int nkv,
                      int hd, const int* row_pos, const int* seq_slot, const int* cu_rows,
                      const int* block_table, int bt_stride, const void* kcache, const void* vcache,
                      float scale, int window, int decode, int max_len, float* workspace,
                      long long workspace_floats, int* tickets, long long tickets_n, const void* k_new,
                      const void* v_new, int ldk, int ldv, const float* cs, int uneven, int pieces,
                      long long piece_stride, hipStream_t stream);

// Floats of workspace lq_attention wants for this launch (0: none).
extern "C" long long lq_attention_workspace(int dtype, int rows, int nh, int nkv, int hd, int block_size,
                                            int decode, int max_len) {
  if (!decode || dtype != LQ_BF16) return 0;
  if (!lq_attention_mfma_accepts(dtype, nh, nkv, hd, block_size, 8, 8, nullptr, nullptr, decode)) return 0;
  return lq_attention_mfma_workspace(rows, nh, nkv, hd, max_len);
}

// A decoding launch shapes its grid by the bound of the lengths rounded up to this many tokens: whoever keeps
// launches for replay (a captured step) needs a new one only when the longest sequence passes a multiple of it.
extern "C" int lq_attention_length_bucket() { return LQ_DECODE_LENGTH_BUCKET; }

// Whether the sequences of a decoding launch differ so much in length (the longest at least half again as long as
// their mean, and 512 tokens or more: below that there is nothing to share out) that the launch does better
// sharing the keys out by the true lengths (`uneven` of lq_attention) than cutting every sequence as if it were
// the longest.  With equal lengths that scheme costs 1 to 3 %, which is why it waits for this answer.
extern "C" int lq_attention_lengths_uneven(const int* lengths, int n) {
  if (lengths == nullptr || n < 2) return 0;
  long long longest = 0, sum = 0;
  for (int i = 0; i < n; ++i) {
    sum += lengths[i];
    if (lengths[i] > longest) longest = lengths[i];
  }
  return longest >= 512 && 2 * (long long)n * longest >= 3 * sum;
}

// For tests, on the host: how many tries the units of an `uneven` decoding launch need to find their split
// length for sequences whose newest positions are pos[0..rows) (0: such a launch does not take that way; -1:
// they would not find it, which must not happen for positions below max_len).
extern "C" int lq_attention_unit_search(const int* pos, int rows, int nkv, int max_len) {
  if (pos == nullptr || rows <= 0 || nkv <= 0 || max_len <= 0) return 0;
  return lq_attention_mfma_unit_search(pos, rows, nkv, max_len);
}

// Whether a decoding launch can take the rotation of q and k and the cache write upon itself
// (lq_attention with k_new, v_new and a cos/sin table; q, k, v are then the unrotated projections).
extern "C" int lq_attention_folds_rope(int dtype, int nh, int nkv, int hd, int block_size) {
  return hd % 64 == 0 && lq_attention_mfma_accepts(dtype, nh, nkv, hd, block_size, 8, 8, nullptr, nullptr, 1);
}

// `decode` != 0 promises one row per sequence; `max_len` is then an upper bound of the
// sequences' lengths after this step (it sizes the split grid, not the result).  `tickets` are
// counters that are zero between launches (a launch leaves them so): one for each row and kv head.
// Launches that share them must not overlap.  `uneven` != 0 says that the sequences of a decoding launch
// differ much in length: its workgroups then share the keys out among themselves by the true lengths
// (the result is the same up to the order of its sums).  `pieces` > 1 (with cs only): q, k_new and v_new
// are float32 partial sums of the projections, `pieces` of them `piece_stride` floats apart, and ldq, ldk
// and ldv count floats; the launch adds them up in order and rounds the sums to the cache's dtype.
extern "C" int lq_attention(const void* q, int ldq, void* out, int ldo, int dtype, int rows, int batch,
                            int nh, int nkv, int hd, const int* row_pos, const int* row_seq,
                            const int* seq_slot, const int* cu_rows, const int* block_table,
                            int bt_stride, const void* kcache, const void* vcache, int block_size,
                            float scale, int window, int decode, int max_len, float* workspace,
                            long long workspace_floats, int* tickets, long long tickets_n, const void* k_new,
                            const void* v_new, int ldk, int ldv, const float* cs, int uneven, int pieces,
                            long long piece_stride, int force_generic, hipStream_t stream) {
  LQ_REQUIRE(rows > 0 && batch > 0, "attention: rows %d and sequences %d must be positive", rows, batch);
  LQ_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0, "attention: %d heads over %d kv heads", nh, nkv);
  LQ_REQUIRE(hd > 0 && block_size > 0 && bt_stride > 0, "attention: bad sizes");
  LQ_REQUIRE(ldq >= nh * hd && ldo >= nh * hd, "attention: a row stride is smaller than its row");
  LQ_REQUIRE(window >= 0, "attention: window %d must not be negative", window);
  LQ_REQUIRE(q && out && row_pos && row_seq && seq_slot && cu_rows && block_table && kcache && vcache,
             "attention: null pointer");
  if (!force_generic && lq_attention_mfma_accepts(dtype, nh, nkv, hd, block_size, ldq, ldo, q, out, decode))
    return lq_attention_mfma(q, ldq, out, ldo, rows, batch, nh, nkv, hd, row_pos, seq_slot, cu_rows,
                             block_table, bt_stride, kcache, vcache, scale, window, decode, max_len,
                             workspace, workspace_floats, tickets, tickets_n, k_new, v_new, ldk, ldv, cs, uneven,
                             pieces, piece_stride, stream);
  LQ_REQUIRE(cs == nullptr && pieces <= 1, "attention: the folded rotation was asked of a launch the matrix-core kernel does not take");
  return lq_attention_generic(q, ldq, out, ldo, dtype, rows, batch, nh, nkv, hd, row_pos, row_seq, seq_slot,
                              block_table, bt_stride, kcache, vcache, block_size, scale, window, stream);
}
