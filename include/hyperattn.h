/*
 * hyperattn.h — C ABI of libhyperattn.so, the MI355X (gfx950) HyperAttention forward path
 * (and the backward of its two attention operators).
 *
 * Every entry point takes raw DEVICE pointers, sizes and strides (in ELEMENTS of the tensor's
 * type unless stated otherwise) and a HIP stream passed as void* (hipStream_t; NULL = the
 * default stream).  The library launches asynchronously on that stream, never synchronises,
 * never allocates or frees device memory and keeps no state between calls: the caller owns
 * every buffer including workspaces (the one exception, ha_bucket_argsort_static, uses a device array
 * that is part of the library's image).  Return value: 0 on success, a negative ha_status for an
 * argument error detected before any launch, or a positive hipError_t from the launch.
 * ha_last_error() returns a thread-local human readable message for the last non-zero status.
 *
 * The reference being replaced is pure Python + Triton; "replaces" below names the reference
 * interface (path relative to the reference checkout : line) each symbol stands in for.
 */
#ifndef HYPERATTN_H
#define HYPERATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HA_ABI_VERSION 6

typedef enum {
  HA_OK = 0,
  HA_ERR_NULL = -1,        /* a required pointer is NULL                                   */
  HA_ERR_DTYPE = -2,       /* dtype is not HA_F16 / HA_BF16 ("Only support fp16 and bf16") */
  HA_ERR_SHAPE = -3,       /* a size is non-positive / not a supported multiple            */
  HA_ERR_HEADDIM = -4,     /* head dim > 128 or not a multiple of 16                        */
  HA_ERR_UNSUPPORTED = -5, /* valid in the reference, not built here (message says what)   */
  HA_ERR_WORKSPACE = -6    /* workspace pointer NULL or too small                           */
} ha_status;

typedef enum { HA_F16 = 0, HA_BF16 = 1 } ha_dtype;
typedef enum { HA_IDX_I32 = 0, HA_IDX_I64 = 1 } ha_idx_type;

int ha_abi_version(void);
const char* ha_last_error(void);

/* ---------------------------------------------------------------------------------------------
 * Angular LSH bucket ids.
 * replaces: AngularLSHTriton.hash_triton -> _angular_lsh -> _angular_lsh_kernel
 *           (src/angular_lsh_triton.py:181-182, :99-145, :14-96)
 * bucket[b,h,i] = gray(sum_j [x[b,h,i,:] . proj[:,j] > 0] << j), gray(v) = v ^ (v >> 1), the closed
 * form of the `perm` table (src/angular_lsh_triton.py:168-173).  The sign is that of the exact dot
 * product (products of fp16/bf16 values are exact; accumulation is in fp64).
 * x: (batch, heads, n, d), last dim contiguous.  proj: (d, r) row-major, shared when
 * proj_stride_b == proj_stride_h == 0, else one matrix per (b,h).  buckets: int32 (batch, heads, n)
 * contiguous.  1 <= r <= 16, d <= 256.
 */
int ha_lsh_hash(const void* x, const void* proj, int32_t* buckets,
                int64_t batch, int64_t heads, int64_t n, int64_t d, int64_t r,
                int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_n,
                int64_t proj_stride_b, int64_t proj_stride_h,
                int dtype, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Segmented stable argsort of small non-negative integer keys (counting sort).
 * replaces: torch.sort(buckets, dim=2, stable=True)[1] at hyper_attention.py:116-117
 * Segment s (0 <= s < num_segments) is keys[seg_offset + s*seg_stride + (0..seg_len)).
 * idx_out[s*seg_len + p] = i such that keys are non-decreasing in p, ties in ascending i;
 * i is LOCAL to the segment (0 <= i < seg_len).  Keys must lie in [0, num_keys); num_keys <= 65536
 * (one 8-bit pass per key byte).  idx_type selects int32 or int64 output.
 * Workspace: ha_bucket_argsort_workspace_bytes(num_segments, seg_len, num_keys) bytes.
 */
int64_t ha_bucket_argsort_workspace_bytes(int64_t num_segments, int64_t seg_len, int64_t num_keys);
int ha_bucket_argsort(const int32_t* keys, void* idx_out, int idx_type,
                      int64_t num_segments, int64_t seg_len, int64_t seg_stride, int64_t seg_offset,
                      int64_t num_keys, void* workspace, int64_t workspace_bytes, void* stream);

/* The same sort without a workspace argument and without any allocation.
 * No counterpart in the reference: it is for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops, harnesses that forbid hipMalloc).  The scratch memory is a device
 * array of HA_SORT_SCRATCH_BYTES inside the library (one copy per GPU, held until the process ends); a
 * sort whose ha_bucket_argsort_workspace_bytes() exceeds it is rejected with HA_ERR_WORKSPACE.  The
 * device of the call is the current device.  All calls on one GPU share the array: calls that overlap
 * on one GPU (different streams or threads) race and must be serialised by the caller.  The first call on a
 * device looks up the array's address and must be made outside stream capture (HA_ERR_UNSUPPORTED
 * otherwise): call it once before capturing.
 */
#define HA_SORT_SCRATCH_BYTES (8 << 20)
int ha_bucket_argsort_static(const int32_t* keys, void* idx_out, int idx_type,
                             int64_t num_segments, int64_t seg_len, int64_t seg_stride, int64_t seg_offset,
                             int64_t num_keys, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Permuting row gather.
 * replaces: indexing(x, indices) (src/attn_utils.py:27-50), the chunk_size < 0 branch; rows
 * [n_idx, n_out) of the output are zero-filled, which is the padding branch (:45-50).
 * out[b,h,s,:] = x[b,h,idx[b,h,s],:].  x (batch,heads,n_src,d) strided, out (batch,heads,n_out,d)
 * contiguous, idx (batch,heads,n_idx) contiguous; elem_bytes is 2 or 4; d*elem_bytes % 16 == 0.
 */
int ha_gather_rows(const void* x, const void* idx, int idx_type, void* out,
                   int64_t batch, int64_t heads, int64_t n_src, int64_t n_idx, int64_t n_out, int64_t d,
                   int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_n,
                   int elem_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Attention operands.  All tensors are addressed as ptr + b*stride_b + h*stride_h + row*stride_n
 * (+ col); the last dim is contiguous.  lse is fp32, addressed lse + b*lse_stride_b + h*lse_stride_h
 * + row.  "Virtual heads": when segs > 1 every (b,h) sequence is cut into `segs` consecutive
 * segments of n_q (resp. n_k) rows that are treated as independent heads; segment g of a q/out/lse
 * sequence starts at row q_seg_offset + g*seg_stride_rows, of a k/v sequence at row
 * k_seg_offset + g*seg_stride_rows.  This is the halves-as-heads view of hyper_attention.py:67-69
 * and the half slicing of :82-84 expressed as index arithmetic.  segs == 1 with zero offsets is the
 * plain case.
 * Limits (HA_ERR_SHAPE / HA_ERR_UNSUPPORTED otherwise): n_q, n_k < 2^24; row strides positive, multiples
 * of 8 elements and below 16 MiB; (n - 1) rows of one head within 4 GiB; tensors 16-byte aligned.
 */
typedef struct {
  const void* q;
  const void* k;
  const void* v;
  void* out;      /* (.., n_q, dv) in dtype                                   */
  float* lse;     /* (.., n_q) fp32                                           */
  int64_t batch, heads, n_q, n_k, d, dv;
  int64_t q_stride_b, q_stride_h, q_stride_n;
  int64_t k_stride_b, k_stride_h, k_stride_n;
  int64_t v_stride_b, v_stride_h, v_stride_n;
  int64_t o_stride_b, o_stride_h, o_stride_n;
  int64_t lse_stride_b, lse_stride_h;
  int64_t segs, seg_stride_rows, q_seg_offset, k_seg_offset;
  /* out and lse of segment g start at row o_seg_offset + g*o_seg_stride_rows of THEIR tensors when
   * o_seg_stride_rows > 0 (a caller that keeps only the rows a call writes, e.g. the second halves of the
   * segments of one level of the causal recursion, packed); 0: they follow q (the two fields above) */
  int64_t o_seg_stride_rows, o_seg_offset;
  int64_t kv_group; /* grouped-query: q head h reads k/v (and k_idx) head h / kv_group; 1 = plain */
  float scale;    /* softmax scale; <= 0 or NaN is an error (callers resolve the default)  */
  int dtype;      /* ha_dtype                                                               */
} ha_attn_operands;

/* Sorted block-diagonal + sampled-column attention, forward.
 * replaces: hyper_attn_func -> HyperAttnFunc.forward -> _hyper_attn_forward -> _fwd_hyper_kernel
 *           (src/hyper_attn_triton.py:895-920, :668-742, :26-192)
 * q_idx / k_idx: permutations of the rows of each (virtual) head, LOCAL row numbers, addressed
 * idx + b*idx_stride_b + h*idx_stride_h + g*n + p*idx_stride_n (g = segment); sampled_idx: sample_size
 * key rows (local), shared by all heads when sampled_stride_h == 0 (sampled_idx == NULL means
 * 0,1,..,sample_size-1, the reference's intended set, src/hyper_attn_triton.py:576-581).
 * PRECONDITION: every entry of sampled_idx lies in [0, n_k).  The list is device memory and is not read
 * by the host, so the library cannot check it: an entry outside the range reads rows of another
 * segment or head (inside a causal recursion: future tokens) or past the tensor, and the backward adds
 * to such rows.  The Python operator layer checks the list on the host before every call.
 * n_q % 128 == 0, n_k % 128 == 0 (:695), sample_size % 128 == 0 (:911); d and dv (value dim, may differ from d: :679,692-693) multiples of 8
 * up to 128: kernels are built for rows of 64 and 128 elements and read narrower rows as they are, the
 * missing columns as zeros.
 * accumulate != 0: out/lse already hold a partial attention over a disjoint key set for every row;
 * the result is merged into them in place (add_self_attentions, src/attn_utils.py:6-24, fused).
 * Residual estimator (no counterpart in the reference, whose sampled loop is src/hyper_attn_triton.py:142-173:
 * un-weighted, duplicates counted; this is the variant of the HyperAttention paper, off unless asked for):
 *   sample_bias != 0: added to the scaled score of every sampled key, e.g. log(n_k / sample_size), which
 *     weights each sample by n_k / sample_size in the soft-max sums;
 *   mask_sampled_in_block != 0: a sampled key that is also among the block keys of the query's tile (its
 *     block, or its smooth window) is left out of the sampled part, so no key is counted twice.  Needs
 *     sampled_pos: for every entry of the sample list the position of that key row in the head's sorted key
 *     order (int32, laid out and strided like sampled_idx; required even when sampled_idx is NULL).
 * Forward only (ha_block_attn_bwd rejects it), d == dv in {64, 128}.
 */
typedef struct {
  ha_attn_operands t;
  const void* q_idx;
  const void* k_idx;
  const void* sampled_idx;
  int idx_type;
  int64_t q_idx_stride_b, q_idx_stride_h, q_idx_stride_n;
  int64_t k_idx_stride_b, k_idx_stride_h, k_idx_stride_n;
  int64_t sampled_stride_b, sampled_stride_h;
  int64_t block_size, sample_size;
  int smooth_block;
  int accumulate;
  const int32_t* sampled_pos;
  float sample_bias;
  int mask_sampled_in_block;
} ha_block_attn_args;

int ha_block_attn_fwd(const ha_block_attn_args* args, void* stream);

/* Exact (flash) attention, forward.
 * replaces: flash_attn_func -> FlashAttnFunc.forward -> _flash_attn_forward -> _fwd_kernel with
 *           bias=None (src/flash_attn_triton.py:995-1012, :795-872, :57-267)
 * Any n_q, n_k >= 1; causal mask row >= col (:177); d, dv multiples of 8 up to 128.
 */
int ha_flash_attn_fwd(const ha_attn_operands* t, int causal, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Backward of the two attention operators: gradients with respect to q, k and v given dout, the
 * gradient of the operator's `out`.  The operands struct is the forward's, with `out` and `lse`
 * holding the forward's results (read only here); a gradient for `lse` is not taken, as in the
 * reference (HyperAttnFunc.backward / FlashAttnFunc.backward ignore it).
 * dq: like q; dk, dv: like k, v, i.e. (batch, heads / kv_group, n_k, d): with grouped queries every
 * query head of a group adds into its key head.  All in dtype, last dim contiguous, written in full
 * (or, with accumulate, added to in full: a caller that differentiates several attention calls on
 * views of the same tensors, like the causal recursion, sums their gradients without extra passes).
 * Segments (segs, seg_stride_rows and the offsets) as in the forward; dout, dq follow q's segment
 * layout, dk, dv that of k, v.  Built for d == dv in {64, 128} (HA_ERR_UNSUPPORTED otherwise).
 * workspace: ha_attn_bwd_workspace_bytes(t, sample_size) bytes (sample_size = 0 for exact attention),
 * 256-byte aligned: two floats per query, and fp32 sums of the sampled keys, cleared by the call.
 */
typedef struct {
  const void* dout;  /* (.., n_q, dv)                          */
  void* dq;
  void* dk;
  void* dv;
  int64_t do_stride_b, do_stride_h, do_stride_n;
  int64_t dq_stride_b, dq_stride_h, dq_stride_n;
  int64_t dk_stride_b, dk_stride_h, dk_stride_n;
  int64_t dv_stride_b, dv_stride_h, dv_stride_n;
  void* workspace;
  int64_t workspace_bytes;
  int accumulate;    /* != 0: dq, dk, dv hold gradients already and the results are added to them   */
} ha_attn_grads;

int64_t ha_attn_bwd_workspace_bytes(const ha_attn_operands* t, int64_t sample_size);

/* replaces: HyperAttnFunc.backward -> _hyper_attn_backward with _bwd_preprocess_do_o_dot,
 *           _bwd_permuted_block_diagonal_kernel, _bwd_sampled_col_kernel
 *           (src/hyper_attn_triton.py:922-945, :745-893, :195-665)
 * Same arguments as ha_block_attn_fwd (accumulate must be 0).  A key that is in a query's block and in
 * the sample list receives both contributions, as it is counted twice in the forward.
 */
int ha_block_attn_bwd(const ha_block_attn_args* args, const ha_attn_grads* grads, void* stream);

/* replaces: FlashAttnFunc.backward -> _flash_attn_backward (src/flash_attn_triton.py:1014-1040,
 *           :875-992) with bias=None.
 */
int ha_flash_attn_bwd(const ha_attn_operands* t, int causal, const ha_attn_grads* grads, void* stream);

/* Merge of two partial attentions.
 * replaces: add_self_attentions (src/attn_utils.py:6-24)
 * rows = batch*heads*n flattened; attn*: (rows, d) with row strides; lse*: fp32 with element
 * strides.  An output may be the very tensor of an input (same pointer and strides) when d is 8, 16,
 * 32, 64, 128, 256 or 512 (HA_ERR_UNSUPPORTED otherwise); partly overlapping tensors are not allowed.
 */
int ha_lse_merge(const void* attn1, const float* lse1, const void* attn2, const float* lse2,
                 void* attn_out, float* lse_out, int64_t rows, int64_t d,
                 int64_t attn1_stride, int64_t attn2_stride, int64_t out_stride,
                 int64_t lse1_stride, int64_t lse2_stride, int64_t lse_out_stride,
                 int dtype, void* stream);

/* The same merge for rows that come in `segs` equal segments of `seg_len` rows, each tensor with its own
 * segment and row strides (in elements; lse and weight arrays: segment strides, rows contiguous): e.g. the
 * second halves of all heads of a (batch, heads, n, d) tensor, in place when the output is the very
 * tensor of an input (same rule as ha_lse_merge).  The weight c of the first input (rounded to dtype first, src/attn_utils.py:21) is used
 * for the merge and, if weight_out is not NULL, written out as fp32: a caller that differentiates the
 * merge needs it (d attn1 = c * d attn, d attn2 = (1 - c) * d attn).  No counterpart in the reference
 * beyond add_self_attentions itself; it serves the causal recursion (hyper_attention.py:86-89).
 */
int ha_lse_merge_segments(const void* attn1, const float* lse1, const void* attn2, const float* lse2,
                          void* attn_out, float* lse_out, float* weight_out,
                          int64_t segs, int64_t seg_len, int64_t d,
                          int64_t attn1_seg_stride, int64_t attn1_row_stride,
                          int64_t attn2_seg_stride, int64_t attn2_row_stride,
                          int64_t out_seg_stride, int64_t out_row_stride,
                          int64_t lse1_seg_stride, int64_t lse2_seg_stride, int64_t lse_out_seg_stride,
                          int64_t weight_seg_stride, int dtype, void* stream);

/* All merges of the causal recursion in one pass (hyper_attention.py:86-89 at every level, i.e. the chain
 * of add_self_attentions calls a row goes through, deepest level first), for a caller that runs the
 * levels itself and keeps their results, as a backward pass needs them.
 * o_leaf, lse_leaf: exact causal attention of the leaves; o_un[j], lse_un[j] (j < levels, 0 = whole
 * sequence): result of the un-masked call of level j.  Every tensor has the layout of the whole
 * (batch_heads, n, d) / (batch_heads, n) contiguous tensors; level j only uses the rows in the second half
 * of each segment of n / 2^j rows.  With packed != 0 the level arrays (o_un[j], lse_un[j], lse_shifted[j])
 * hold those rows only, the second halves of the level's segments one after the other: (batch_heads, n/2, d)
 * and (batch_heads, n/2) (what a call writes with o_seg_stride_rows = n / 2^(j+1), o_seg_offset = 0).
 * out, lse_out: the merged result (not in place).
 * If leaf_shifted is not NULL, lse_shifted[j] (second halves) and leaf_shifted (all rows) receive
 * lse - log(w), w the total weight the merges give that call's result in `out`: handing a call's backward
 * this log-sum-exp together with the gradient of `out` equals handing it its own log-sum-exp and w times
 * the gradient (weights carry no gradient, src/hyper_attn_triton.py:922-945).
 */
int ha_lse_merge_levels(const void* o_leaf, const float* lse_leaf, const void* const* o_un,
                        const float* const* lse_un, float* const* lse_shifted, float* leaf_shifted,
                        void* out, float* lse_out, int levels, int64_t batch_heads, int64_t n, int64_t d,
                        int dtype, int packed, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Whole forward pass of the module for (batch, heads, n, d) tensors, one call, no host
 * synchronisation and no tensor copies.
 * replaces: HyperAttention.forward / forward_no_causal_mask (hyper_attention.py:25-132) for the
 * shapes where every recursion level has an even length (n = leaf_len * 2^levels); other shapes
 * are composed by the caller from the operators above.
 * proj: (d, r) in dtype, r = lsh_num_projs <= 16 (the reference takes any r, padded to 16 slots,
 * src/angular_lsh_triton.py:116-144).  d, dv: multiples of 8 up to 128.  Workspace:
 * ha_forward_workspace_bytes(args) bytes, 256-byte aligned; it holds the bucket ids, the per-unit orders
 * and counts of the one ranking (r <= 8; above, a sort per level with its digit passes) and the int32
 * orders of every hashed level.  sampled_idx: int32 key rows local to each un-masked call (NULL = first
 * sample_size rows), shared by all heads and levels; PRECONDITION as for ha_block_attn_fwd, with n_k the
 * key length of the shortest hashed level (n / 2^levels halvings down to the last length >= min_seq_len).  out (batch,heads,n,dv) dtype, lse
 * (batch,heads,n) fp32.  kv_heads divides heads (grouped-query: q head h reads kv head
 * h / (heads/kv_heads)); k and v are (batch, kv_heads, n, d).
 * q/k/v strides in elements, last dim contiguous; a tensor whose three strides are all zero is
 * contiguous.  This takes the permuted views of the reference's callers
 * (chatglm_fast_attention.py:42-58: (sq, b, np, hn) tensors seen as (b, np, sq, hn)) without a copy.
 */
typedef struct {
  const void* q;
  const void* k;
  const void* v;
  const void* proj;
  const int32_t* sampled_idx;
  void* out;
  float* lse;
  int64_t batch, heads, kv_heads, n, d, dv;
  int64_t lsh_num_projs, block_size, sample_size, min_seq_len;
  int smooth_block;
  int causal;
  float scale;
  int dtype;
  void* workspace;
  int64_t workspace_bytes;
  int64_t q_stride_b, q_stride_h, q_stride_n;
  int64_t k_stride_b, k_stride_h, k_stride_n;
  int64_t v_stride_b, v_stride_h, v_stride_n;
} ha_forward_args;

int64_t ha_forward_workspace_bytes(const ha_forward_args* args);
int ha_forward(const ha_forward_args* args, void* stream);

/* The first stage of ha_forward alone: bucket ids of q and k (one launch) and the stable bucket order of the
 * query and key segment of every hashed level (one ranking of the rows, one placement launch for all
 * levels), written into the workspace.
 * replaces: the lsh.hash + torch.sort pairs of every level of the recursion (hyper_attention.py:112-117
 * under :51-96) for a caller that runs the levels itself, e.g. to keep what a backward pass needs.
 * For level j (0 = whole sequence; the only one without a causal mask) q_idx_offset[j] / k_idx_offset[j]
 * receive the byte offsets into the workspace of int32 arrays (batch, heads * 2^j, half) and
 * (batch, kv_heads * 2^j, half) of rows local to the level's query segment (second halves) and key segment
 * (first halves), or -1 where the level is exact (its half is shorter than min_seq_len).  Both arrays must
 * hold 48 entries; *num_levels receives the number of levels.  Only q, k, proj, the sizes, dtype, causal,
 * min_seq_len, lsh_num_projs, the strides and the workspace of `args` are read.
 */
int ha_forward_sort(const ha_forward_args* args, int64_t* q_idx_offset, int64_t* k_idx_offset, int* num_levels,
                    void* stream);

/* ---------------------------------------------------------------------------------------------
 * Measurement aid (no counterpart in the reference, not on the forward path): single-purpose loops that
 * price the board's power limit.  `workgroups` workgroups of 256 threads each run `trips` trips of four
 * half-step blocks (8 large MFMAs each, where the kind has them): HA_PROBE_MFMA on register operands only,
 * HA_PROBE_LDS_MFMA with the attention kernels' LDS operand reads, HA_PROBE_SOFTMAX the soft-max arithmetic of
 * the blocks alone, HA_PROBE_BLOCK all of it, HA_PROBE_BLOCK_WIDE all of it with 16 MFMAs per block (the d = 128 ratio).  One
 * trip of one workgroup is 4 waves * 4 blocks * 8 (16) MFMAs of 32768 flops.
 * sink: 256 floats of device memory (never written in practice).  bench.py times these loops with the board
 * power sampled beside them.
 */
enum { HA_PROBE_MFMA = 0, HA_PROBE_LDS_MFMA = 1, HA_PROBE_SOFTMAX = 2, HA_PROBE_BLOCK = 3, HA_PROBE_BLOCK_WIDE = 4 };
int ha_power_probe(int kind, int64_t trips, int workgroups, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HYPERATTN_H */
