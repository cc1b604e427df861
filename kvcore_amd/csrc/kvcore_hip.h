// C interface of the gfx950 kernel library.  Every function launches on the given
// stream and returns at once; 0 means the launch was accepted, a negative value
// means the arguments were refused (kvc_last_error() holds the reason) and nothing
// was launched.  Pointers are device pointers unless named host_*.
//
// dtype codes: 0 = float32, 1 = bfloat16.  "dt" in a comment means that type.
#pragma once

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* kvc_stream;

const char* kvc_last_error(void);
int kvc_version(void);
// Compute units of the current device: what the launch plans of the attention kernels count
// blocks against.
int kvc_compute_units(void);
// The variant that this thread's last launch of a kernel family took, as a short text such as
// "prefill_attention_kernel<128,1,8,8> x1" (head size, column tiles, key blocks a tile, waves,
// then the number of splits) or "rope_kv_write_tile_kernel"; "" if the family has not been
// launched.  Families: 0 attention over portions of prompts, 1 rotation with the cache write.
const char* kvc_last_variant(int family);

// Measurement only (peaks.hip).  kvc_peak_read: `blocks` blocks of 256 threads read `bytes` bytes
// of `buffer` once with 16-byte loads and store nothing (`sink`: four bytes that are practically
// never written); timed by the caller over buffers too large for the caches, it gives the read
// bandwidth that a kernel can reach at all.  kvc_peak_mfma_bf16: every wave of `blocks` blocks
// of four issues `rounds` x 4 independent 32x32x16 bfloat16 matrix instructions on operands in
// registers (2 x 32 x 32 x 16 flops each) and stores one float a thread into `out`.
int kvc_peak_read(const void* buffer, int64_t bytes, int blocks, void* sink, kvc_stream stream);
int kvc_peak_mfma_bf16(float* out, int blocks, int rounds, kvc_stream stream);

// residual[t, :] = float(table[ids[t], :]) * scale; an id outside [0, V) gives a NaN row.
int kvc_embed(float* residual, const void* table, const int32_t* ids, int T, int H, int V,
              int dtype, float scale, kvc_stream stream);

// What a head may do to its logits [S, V] (float32, rows row_stride apart) after the product,
// in place: x += bias[v] (bias of bias_dtype, or null); x = soft_cap * tanh(x / soft_cap) when
// soft_cap > 0; x *= scale.
int kvc_logits_finish(float* logits, int S, int V, int64_t row_stride, const void* bias,
                      int bias_dtype, float soft_cap, float scale, kvc_stream stream);

// Every element of the pages pages[i * page_stride], i < n, in all `outer` planes of a cache
// group's storage [outer, num_pages, page_elems] (elements of elem_bytes = 2 or 4) becomes the
// bit pattern `bits` (its low 16 bits for 2-byte elements): zeros, or a NaN that makes a read
// of a slot nobody wrote show in the logits.  The null page (0) and ids outside the pool are
// skipped.  Reference: kvcore/model/model_runner.py:646-657 zeroes new blocks with index_fill_.
int kvc_fill_pages(void* storage, const int32_t* pages, int page_stride, int n, int outer,
                   int num_pages, int64_t page_elems, int elem_bytes, uint32_t bits, kvc_stream stream);

// out[i] = mean + std * z_i for i < n, out of dtype: z_i is a standard normal variate that is a
// function of (seed_lo, seed_hi, i) alone, worked out in single float32 operations that a host
// program can repeat bit for bit (see random_fill.hip).
int kvc_fill_normal(void* out, int64_t n, int dtype, uint32_t seed_lo, uint32_t seed_hi, float mean,
                    float std, kvc_stream stream);

// residual += delta (skipped when delta is null); out = weight * residual *
// rsqrt(mean(residual^2) + eps), rounded to dt.  residual stays float32.
int kvc_add_rmsnorm(void* out, float* residual, const void* delta, const float* weight,
                    float eps, int T, int H, int dtype, kvc_stream stream);
// The same with the pending output given as float32 partial sums [slices, T, H] of a product
// cut along K (see kvc_gemm_mid_bf16, mode 2) and an optional bfloat16 bias [H]: the slices
// are added up in their order, then into the residual.  H a multiple of 8, at most 16384.
int kvc_add_slices_rmsnorm(void* out, float* residual, const float* partial, int slices,
                           const void* bias, const float* weight, float eps, int T, int H, int dtype,
                           kvc_stream stream);

// out = weight * x * rsqrt(mean(x^2) + eps) on rows of dt (no residual), row strides given.
int kvc_rmsnorm(void* out, const void* x, const float* weight, float eps, int T, int H,
                int64_t x_stride, int64_t out_stride, int dtype, kvc_stream stream);

// residual += delta, nothing else.
int kvc_residual_add(float* residual, const void* delta, int T, int H, int dtype,
                     kvc_stream stream);

// out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i].
int kvc_silu_mul(void* out, const void* gate_up, int T, int I, int dtype, kvc_stream stream);

// out[s, :] = in[rows[s], :]; `in` may be float32 (in_dtype 0) while out is dt.
int kvc_gather_rows(void* out, const void* in, const int32_t* rows, int S, int H, int in_dtype,
                    int out_dtype, kvc_stream stream);

// out = float(in) elementwise (n values).
int kvc_to_float(float* out, const void* in, int64_t n, int dtype, kvc_stream stream);

// cos/sin[t, j] of the angle float(positions[t]) * inv_freq[j], j < half.
int kvc_rope_table(float* cos_out, float* sin_out, const int32_t* positions,
                   const float* inv_freq, int T, int half, kvc_stream stream);

// kv_slot[t] = page * page_size + position % page_size, where page = table[slots[
// token_req[t]], position / page_size]; -1 when the table holds no page there, -2 for a
// padding token (token_req < 0).
int kvc_kv_slots(int32_t* kv_slot, const int32_t* positions, const int32_t* token_req,
                 const int32_t* slots, const int32_t* table, int table_stride, int T,
                 int page_size, int num_pages, kvc_stream stream);

// Rotates the first rot_dim elements of every q and k head of qkv [T, (nh+2nkv)*d] in
// place (pairs (j, j+rot_dim/2), or (2j, 2j+1) when interleaved), then, when write_kv is
// set and kv_slot[t] >= 0, stores the rotated k and the v of token t at that slot:
//   k_cache[page, kv_head, offset, :] and v_cache[page, kv_head, :, offset]
//   (V pages keep the keys contiguous: the layout the matrix cores read).
// Tokens with kv_slot == -2 are left alone.  Without rotate_q the q heads stay as they are
// (for a consumer that rotates them itself, as kvc_prefill_attention can).
int kvc_rope_kv_write(void* qkv, void* k_cache, void* v_cache, const float* cos_tab,
                      const float* sin_tab, int rot_dim, int interleaved, const int32_t* kv_slot,
                      int T, int nh, int nkv, int d, int page_size, int write_kv, int rotate_q,
                      int dtype, kvc_stream stream);

// Attention of every token over its request's cache: token t at position p sees keys
// max(0, p - window + 1) .. p (window <= 0: all), read through the block table.
// q is [T, nh, d] with q_stride elements between tokens; out is [T, nh*d].
int kvc_paged_attention(void* out, const void* q, int64_t q_stride, const void* k_cache,
                        const void* v_cache, const int32_t* table, int table_stride,
                        const int32_t* positions, const int32_t* token_req,
                        const int32_t* slots, int T, int nh, int nkv, int d, int page_size,
                        int num_pages, float scale, int window, int dtype, kvc_stream stream);

// The same attention for bfloat16 steps of single tokens on the matrix cores, a block of
// several waves per (token, kv head, split), which also does what kvc_rope_kv_write does for
// its token: qkv rows are [nh q heads | nkv k heads | nkv v heads]; the first rot_dim elements
// of every q head (and of the k head) are rotated by cos/sin [T, rot_dim / 2] on the way in
// (rot_dim 0: taken as they are) and qkv itself is left unchanged; with write_kv the
// token's key and value are stored in their cache slot and attended to (without write_kv
// the cache must already hold them).  nsplit > 1 needs part_o [T, nh, nsplit, d] and part_ml
// [T, nh, nsplit, 2] float32; a second kernel combines the splits (a "last block combines"
// scheme needs device-scope fences, which on this chip write back and invalidate a whole L2
// slice per block and cost more than the launch they save).
// token_rows [T], if not null, holds slots[token_req[t]] (-1 for padding) and saves the
// kernel one dependent load.
// kvc_decode_attention_supported tells whether a shape is served (else use
// kvc_paged_attention); kvc_decode_attention_waves how many waves share a block's key range.
// kvc_decode_attention_max_table: the widest block table (entries per request) whose page ids
// for one split still fit in a block's LDS; a wider one is refused, so engines check it when
// they are built.
int kvc_decode_attention_supported(int nh, int nkv, int d, int page_size, int dtype);
int kvc_decode_attention_waves(int nh, int nkv, int d);
int kvc_decode_attention_max_table(int nh, int nkv, int d);
int kvc_decode_attention(void* out, void* part_o, void* part_ml, const void* qkv,
                         int64_t qkv_stride, void* k_cache, void* v_cache, const int32_t* table,
                         int table_stride, const int32_t* positions, const int32_t* token_req,
                         const int32_t* slots, const int32_t* token_rows, const float* cos_tab,
                         const float* sin_tab, int rot_dim, int interleaved, int write_kv, int T,
                         int nh, int nkv, int d, int page_size, int num_pages, float scale,
                         int window, int nsplit, kvc_stream stream);

// The same attention for bfloat16 portions of prompts on the matrix cores: a block per
// (tile of a request's tokens, kv head), keys staged through LDS.  q_start [R+1] bounds
// each request's tokens in the flattened batch; slots [R] names its block-table row;
// positions must rise by one along a request's tokens.  With nsplit > 1 the keys of every
// tile are dealt to that many blocks (for few query rows against many keys) and a second
// kernel joins their results; part_o [T*nh*nsplit, d] and part_ml [T*nh*nsplit, 2] float32
// are its workspace.  With cos_tab and sin_tab [T, rot_dim / 2] the queries come unrotated
// and are rotated on their way in, as kvc_rope_kv_write would have (rot_dim a multiple of 64,
// or of 32 when interleaved); without, they are taken as they are.
int kvc_prefill_attention_supported(int nh, int nkv, int d, int page_size, int dtype);
int kvc_prefill_attention(void* out, const void* q, int64_t q_stride, const void* k_cache,
                          const void* v_cache, const int32_t* table, int table_stride,
                          const int32_t* positions, const int32_t* q_start, const int32_t* slots,
                          int T, int R, int nh, int nkv, int d, int page_size, int num_pages,
                          float scale, int window, void* part_o, void* part_ml, int nsplit,
                          const float* cos_tab, const float* sin_tab, int rot_dim, int interleaved,
                          kvc_stream stream);

// C[M, N] = A[M, K] * W[N, K]^T (+ bias[N]) in float32 with float32 products and sums;
// each element is one running sum over k = 0..K-1, whatever M is.
int kvc_gemm_f32(float* C, const float* A, const float* W, const float* bias, int M, int N,
                 int K, int64_t lda, int64_t ldc, kvc_stream stream);

// The same product for 17 to 192 rows, where the waves of a block share the rows of A through
// LDS (K a multiple of 512).  mode 0: C = A W^T (+ bias), float32 (out_dtype 0) or bfloat16
// (1).  mode 1: C[M, N] = silu(A Wg^T + bg) * (A Wu^T + bu) in bfloat16, W [2N, K] holding Wg
// then Wu.  mode 2: narrow outputs are cut along K into kvc_gemm_mid_slices(N, K) slices and
// only their float32 partial sums are stored, partial [slices, M, N] (no bias); the kernel
// that consumes them adds them up in slice order.  mode 3: as mode 0, but cut along K like
// mode 2 when `partial` is given, with a second kernel that sums the slices.  With `packed` W
// is what kvc_pack_weight made of the matrix (the same sums, read in contiguous kilobytes).
int kvc_gemm_mid_slices(int N, int K);
int kvc_gemm_mid_bf16(void* C, void* partial, const void* A, const void* W, const void* bias, int M,
                      int N, int K, int64_t lda, int64_t ldc, int out_dtype, int mode, int packed,
                      kvc_stream stream);

// C[M, N] = A[M, K] * W[N, K]^T (+ bias[N]) for M <= 64 rows of bfloat16 on the matrix
// cores, float32 sums, weights streamed once; C is float32 (out_dtype 0) or bfloat16 (1).
// K and lda must be multiples of 8, A and W 16-byte aligned.  With `packed` W is what
// kvc_pack_weight made of the matrix (N a multiple of 16, K of 64): the same sums in the same
// order, read in contiguous kilobytes.
int kvc_gemm_skinny_bf16(void* C, const void* A, const void* W, const void* bias, int M, int N,
                         int K, int64_t lda, int64_t ldc, int out_dtype, int packed,
                         kvc_stream stream);

// dst = src [N, K] bfloat16 in tiles of 16 rows x 32 columns of 1 KB each, the tiles of 16
// rows one after the other along K (N a multiple of 16, K of 64): element (n, k) goes to
// ((n / 16) * (K / 32) + k / 32) * 512 + (n % 16) * 32 + k % 32.  That is the order in which
// the products for few rows read the weights, whose loads then are one contiguous kilobyte
// instead of 64 bytes from each of 16 rows.
int kvc_pack_weight(void* dst, const void* src, int N, int K, kvc_stream stream);

// C[M, N] = silu(A Wg^T + bg) * (A Wu^T + bu) for M <= 64 rows of bfloat16, where Wg is rows
// 0..N-1 of W[2N, K] and Wu rows N..2N-1 (bias[2N] likewise): the gated feed-forward's first
// product with its activation, both factors rounded to bfloat16 before the activation as the
// two-kernel form stores them.  C is bfloat16.
int kvc_gemm_skinny_silu_mul_bf16(void* C, const void* A, const void* W, const void* bias, int M,
                                  int N, int K, int64_t lda, int64_t ldc, int packed,
                                  kvc_stream stream);

// The same products with the RMS norm of the rows folded in, for steps of at most 16 tokens,
// so that no separate norm kernel runs between them:
//  - in_ss [M, in_parts] (or null): A holds rows with the norm's gain applied but not yet
//    normalised; row m's sums are multiplied by rsqrt(sum_p in_ss[m, p] / in_width + in_eps)
//    before bias (and activation);
//  - residual [M, ldr] float32 (or null; not with gated): residual += product (+ bias); C
//    receives bfloat16(residual * gain[n]) and out_ss [M, blocks] the new residual's sums of
//    squares per block of columns, blocks = kvc_gemm_skinny_blocks(N, K, 0, packed): the in_ss of the
//    product that consumes C.
// gated = 1 is kvc_gemm_skinny_silu_mul_bf16's product (N = the gate's rows).
int kvc_gemm_skinny_blocks(int N, int K, int gated, int packed);
int kvc_gemm_skinny_fused_bf16(void* C, const void* A, const void* W, const void* bias, int M, int N,
                               int K, int64_t lda, int64_t ldc, int gated, const float* in_ss,
                               int in_parts, int in_width, float in_eps, float* residual,
                               int64_t ldr, const float* gain, float* out_ss, int packed,
                               kvc_stream stream);

// table[triples[3i], triples[3i+1]] = triples[3i+2] for i < n.
int kvc_table_update(int32_t* table, int table_stride, int table_rows, const int32_t* triples,
                     int n, kvc_stream stream);

// out[s] = index of the largest logit of row s (the lowest index among equals).  With a
// workspace (part_val, part_idx: part_capacity >= S * ceil(V / 8192) entries each) long rows
// are searched by several blocks; the pointers may be null.
int kvc_argmax(int32_t* out, const float* logits, int S, int V, int64_t row_stride,
               float* part_val, int32_t* part_idx, int part_capacity, kvc_stream stream);

// kvc_argmax for callers that cannot allocate device memory and bring no workspace (code
// under HIP graph capture, tight serving loops, harnesses that forbid allocation).  It has no
// counterpart in the reference.  The partial results of long rows live in a static device
// array of kvc_argmax_static_capacity() = 16384 entries (128 KB that every GPU the library
// runs on holds until the process ends); S * ceil(V / 8192) beyond that is refused with an
// error, rows of at most 8192 values need no partial results and are never refused.  The call
// allocates and frees nothing, on the device or through any library.  The array keeps the last
// call's contents; nothing in it has to start at zero, since every entry that is read was
// written earlier in the same call.  All calls on one GPU share that GPU's array: calls that
// overlap there (different streams or threads) race, calls on one stream do not.  The results
// equal kvc_argmax's.
int kvc_argmax_static_capacity(void);
int kvc_argmax_static(int32_t* out, const float* logits, int S, int V, int64_t row_stride,
                      kvc_stream stream);

// Per row s: temperature[s] < 1e-5 gives the argmax; otherwise
// argmax_v(logits[v] / temperature - log(e_v)), e_v exponential noise keyed by
// (seed_lo[s], seed_hi[s], index[s], v), over the entries that top_k[s] (<= 0: all) and
// top_p[s] (>= 1: all) keep.  With a workspace of kvc_sample_workspace_words(S, V) 64-bit
// words (0: rows too short to gain) every row is dealt to several blocks, which gives the
// same draws; it need not be cleared.  filters: bit 0, some row has a top_k; bit 1, some row
// has a top_p < 1 (passes that no row needs are left out; 3 is always right).
int kvc_sample_workspace_words(int S, int V);
int kvc_sample(int32_t* out, const float* logits, int S, int V, int64_t row_stride,
               const float* temperature, const int32_t* top_k, const float* top_p,
               const uint32_t* seed_lo, const uint32_t* seed_hi, const uint32_t* index,
               void* workspace, int64_t workspace_words, int filters, kvc_stream stream);

#ifdef __cplusplus
}
#endif
