/* flyhip -- C ABI of the MI355X (gfx950) kernels for the Scatterbrain-local attention path and
 * the block-sparse matmul / row-op path of HazyResearch/fly.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller (PyTorch in the shipped host code);
 *     the library never allocates, frees or synchronises; work is enqueued on `stream`
 *     (a hipStream_t passed as void*, NULL = default stream);
 *   - entry points return 0 on success and a negative code otherwise; the message is
 *     available from flyhip_last_error() (thread-local);
 *   - dtype: 0 = float32, 1 = bfloat16, 2 = float16 (storage type; accumulation is fp32);
 *   - strides are in elements;
 *   - a stream that is under capture into a HIP graph is refused (negative return, message): the
 *     launchers do work on first use that is not a stream operation, so calls of this library
 *     are to be made eagerly.
 *
 * "ref:" comments name the interface in the reference checkout that each entry point replaces.
 */
#ifndef FLYHIP_H
#define FLYHIP_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

enum { FLYHIP_F32 = 0, FLYHIP_BF16 = 1, FLYHIP_F16 = 2 };
enum { FLYHIP_SB_CHUNK = 64 };           /* keys per feature chunk / key tile */

int flyhip_version(void);
const char* flyhip_last_error(void);

/* ------------------------------------------------------------------------------------------
 * Scatterbrain-local attention (ref: src/models/attention/sblocal_attention.py:43-137)
 * ---------------------------------------------------------------------------------------- */

/* Sizes of the caller-allocated scratch for one problem: n_chunks = ceil(S/64), the number n_split
 * of partial K'^T V reductions per (batch, head), and the number n_parts of pieces the band of
 * every 64-query tile is split into by flyhip_sblocal_fwd (1 = no partial workspace needed). */
int flyhip_sb_plan(int B, int H, int T, int S, int local_context,
                   int* n_chunks, int* n_split, int* n_parts);
/* The same for a known kernel choice: E the padded head dim, mh the padded projection rows, dtype the code of the
 * inputs.  n_split then accounts for how many workgroups of that key pass a compute unit holds (one for fp32 inputs on
 * the bf16-piece kernels, two otherwise); n_chunks and n_parts as above.  (No counterpart in the reference: launch
 * geometry.) */
int flyhip_sb_plan_for(int B, int H, int T, int S, int local_context, int E, int mh, int dtype,
                       int* n_chunks, int* n_split, int* n_parts);

/* Key-side pass.  Replaces feature_map.forward_keys (ref: feature_maps_sb.py:51-82, key branch),
 * the masking of padded keys (sblocal_attention.py:83-85) and the global reductions
 * linear_attention / linear_attention_normalization (ref: scatterbrain_utils.py:18-22,48-52:
 * K'^T V and sum_s K').
 *   k (B,S,H,E), v (B,S,H,D) addressed through strides (batch, head, seq); innermost contiguous
 *   proj (mh, E) fp32 row-major, rows >= mh_valid ignored (zero rows); E = D in {32,64,128},
 *   m = 2*mh in {32,64,128,256}
 *   key_lengths (B) int64 or NULL
 * outputs (fp32 unless noted):
 *   kfeat       (B,H,n_chunks*64,m)  positive random features of every key, stabilised per chunk;
 *                                    opaque scratch in the element type of k (fp32, or bf16 in the
 *                                    k-slot order of the bf16 MFMA) -- only flyhip_sblocal_fwd reads it
 *   chunk_scale (B,H,n_chunks)       log-stabiliser each chunk of kfeat was written with
 *   kv (B,H,m,D), ksum (B,H,m), kmax (B,H)  global reductions in units of exp(kmax)
 * scratch: kv_part (B,H,n_split,m*(D+1)), part_max (B,H,n_split).
 * Optional query side (q may be NULL; needed when flyhip_sblocal_fwd runs with n_parts > 1, where
 * several workgroups share a query tile): q (B,T,H,E) via strides -> qfeat (B,H,T,m) fp32, the
 * query features exp(+-sqrt(t) P q - rowmax) (ref: softmax_kernel with is_query=True,
 * src/models/attention/feature_maps_sb.py:51-82,148-151), and q_lsq (B,H,T) fp32, their log-scale
 * -t|q|^2/2 + rowmax - log(m)/2.  With q given, kv / ksum / kmax are NOT written: the partial
 * reductions (kv_part, part_max) are combined inside flyhip_sblocal_fwd's launch instead, which
 * saves a launch on problems this small.
 * bfloat16 inputs: vt (B,H,n_chunks*64,D) bf16 and kvt (B,H,2,D,m) bf16 (K'^T V in two bf16 pieces), opaque scratch for
 * flyhip_sblocal_fwd -- V per 32-key tile and K'^T V, transposed into the operand order of the bf16
 * MFMA.
 * float inputs: vt may be NULL (all products on the fp32 matrix pipe, kfeat holds fp32 features).
 * With vt given -- B*H*n_chunks*2*(128*E + 192*D) bytes suffice, 16-byte aligned -- the key pass writes
 * per 32-key tile an image of K and V^T split into bfloat16 pieces there, and into kfeat (same
 * byte size as the fp32 features) an image of the features split into two pieces; passing the same
 * vt to flyhip_sblocal_fwd then runs the band on the bf16 matrix pipe with fp32-level accuracy
 * (features are rounded to 17 significant bits where they are formed, V to 16 in both of its products).  kvt is unused for float. */
int flyhip_sb_kv_reduce(const void* k, const void* v, const float* proj, const int64_t* key_lengths,
                        void* kfeat, float* chunk_scale, float* kv_part, float* part_max,
                        float* kv, float* ksum, float* kmax,
                        const void* q, float* qfeat, float* q_lsq, int T,
                        int64_t q_sb, int64_t q_sh, int64_t q_ss, void* vt, void* kvt,
                        int B, int H, int S, int E, int D, int mh, int mh_valid, int n_split,
                        int64_t k_sb, int64_t k_sh, int64_t k_ss,
                        int64_t v_sb, int64_t v_sh, int64_t v_ss,
                        float softmax_temp, int dtype, void* stream);

/* Fused query-side pass.  Replaces feature_map.forward_queries, both local_dot_product calls, the
 * joint normalisation and local_weighted_average + combine (ref: sblocal_attention.py:78,90-122;
 * fast_transformers.local_product).  Consumes the outputs of flyhip_sb_kv_reduce.
 *   q (B,T,H,E), out (B,T,H,D) via strides; log_norm (B,H,T) fp32 = the reference's
 *   log_normalization; local_context = lc (band -(lc/2) <= s - i < (lc+1)/2).
 *   n_parts from flyhip_sb_plan (any value in [1,64] is valid); when > 1, part_ws is scratch of
 *   B*H*ceil(T/64)*n_parts*64*(D+5) floats and qfeat / q_lsq are the query-side outputs of
 *   flyhip_sb_kv_reduce for the same q; with n_parts == 1 all three may be NULL (the kernel forms
 *   the query features itself).  vt / kvt: the scratch of flyhip_sb_kv_reduce (float inputs: vt as
 *   it was passed there, NULL or the piece images; kvt NULL).
 *   With n_parts > 1 the key pass has left its partial reductions uncombined: pass its kv_part,
 *   part_max and n_split; extra workgroups of the band kernel's launch combine them into kv / ksum /
 *   kmax (written here, read by the merge kernel that finishes the tiles).  With n_parts == 1 they
 *   are ignored and kv / ksum / kmax are inputs. */
int flyhip_sblocal_fwd(const void* q, const void* k, const void* v, const float* proj,
                       const void* kfeat, const float* chunk_scale,
                       float* kv, float* ksum, float* kmax,
                       const float* qfeat, const float* q_lsq, const void* vt, const void* kvt,
                       const float* kv_part, const float* part_max, int n_split,
                       const int64_t* key_lengths, void* out, float* log_norm,
                       float* part_ws, int n_parts,
                       int B, int H, int T, int S, int E, int D, int mh, int mh_valid,
                       int local_context,
                       int64_t q_sb, int64_t q_sh, int64_t q_ss,
                       int64_t k_sb, int64_t k_sh, int64_t k_ss,
                       int64_t v_sb, int64_t v_sh, int64_t v_ss,
                       int64_t o_sb, int64_t o_sh, int64_t o_ss,
                       float softmax_temp, int dtype, void* stream);

/* The whole forward of Scatterbrain-local attention in one call (ref: SBLocalAttention.forward,
 * src/models/attention/sblocal_attention.py:73-122, for causal = False, attn_mask = None, eps = 0, no dropout):
 * flyhip_sb_kv_reduce followed by flyhip_sblocal_fwd on ONE caller-provided workspace, which the library divides
 * into the scratch of both calls (for float inputs that includes the tile images of the key pass, so the band
 * kernel runs on the bf16 matrix pipe).  flyhip_sb_workspace_bytes gives its size for a problem (E = D: padded
 * head dim, mh: padded projection rows; -1 for bad arguments).  The workspace must be aligned to 256 bytes; its
 * contents need no initialisation and mean nothing between calls; one call at a time may use it.
 * flags: 0, or FLYHIP_SB_EXACT_FP32 -- float inputs then take the fp32 matrix pipe for every product (no bf16
 * pieces, V and the features not rounded: about 1e-6 of the float64 result instead of 5e-6, at 1.6 times the
 * time); pass the same flags to both functions.
 * dropout_p in [0, 1), dropout_seed: dropout of the exact weights exp(QK - log_normalization) as in
 * sblocal_attention.py:119 (the normaliser and the low-rank part see none).  No mask is stored: whether the weight of
 * (query i, key s) of (batch b, head h) is kept is a hash of (seed, (b H + h) T + i, s) -- written out at
 * flyhip_bs_attn_dropout, with L = T -- and kept weights are scaled by 1 / (1 - p); flyhip_sblocal_bwd_pieces forms
 * the same mask from the same seed.  float32 inputs with head dims up to
 * 64 and up to 128 features (the kernels on bf16 pieces), not with FLYHIP_SB_EXACT_FP32; 0 = no dropout.
 * Arguments otherwise as for flyhip_sb_kv_reduce / flyhip_sblocal_fwd.
 * float16 tensors: dtype = 0 | (2 << 8) -- float32 arithmetic on operand images (not with FLYHIP_SB_EXACT_FP32; head dims
 * up to 64, up to 128 features) with q, k, v read and out written as float16: the kernels widen what they load and round
 * what they store. */
#define FLYHIP_SB_EXACT_FP32 1
int64_t flyhip_sb_workspace_bytes(int B, int H, int T, int S, int E, int mh, int local_context, int dtype, int flags);
int flyhip_sblocal_forward(const void* q, const void* k, const void* v, const float* proj,
                           const int64_t* key_lengths, void* out, float* log_norm,
                           void* workspace, int64_t workspace_bytes,
                           int B, int H, int T, int S, int E, int D, int mh, int mh_valid, int local_context,
                           int64_t q_sb, int64_t q_sh, int64_t q_ss,
                           int64_t k_sb, int64_t k_sh, int64_t k_ss,
                           int64_t v_sb, int64_t v_sh, int64_t v_ss,
                           int64_t o_sb, int64_t o_sh, int64_t o_ss,
                           float softmax_temp, int dtype, int flags,
                           float dropout_p, uint64_t dropout_seed, void* stream);

/* flyhip_sblocal_fwd for callers that cannot allocate device memory -- tight serving loops, harnesses
 * that forbid hipMalloc.  It has no counterpart in the reference.
 * Same arguments and results as flyhip_sblocal_fwd except that there is no part_ws: the partial
 * outputs of the parts of a query tile go to a fixed 16 MiB array inside the library (one copy per
 * GPU, held until the process ends).  The call allocates and frees nothing.  It fails with a
 * message when B*H*ceil(T/64)*n_parts*64*(D+5) exceeds 4 Mi floats (n_parts > 1 only; with
 * n_parts == 1 no scratch is used).  All calls on one GPU share that array: calls that overlap in
 * time on one GPU (different streams or threads) race.  Its address is looked up on the first call
 * on each device, with that device current.  (Like every entry point of this library it refuses a stream
 * that is under graph capture.) */
int flyhip_sblocal_fwd_static(const void* q, const void* k, const void* v, const float* proj,
                              const void* kfeat, const float* chunk_scale,
                              float* kv, float* ksum, float* kmax,
                              const float* qfeat, const float* q_lsq, const void* vt, const void* kvt,
                              const float* kv_part, const float* part_max, int n_split,
                              const int64_t* key_lengths, void* out, float* log_norm,
                              int n_parts,
                              int B, int H, int T, int S, int E, int D, int mh, int mh_valid,
                              int local_context,
                              int64_t q_sb, int64_t q_sh, int64_t q_ss,
                              int64_t k_sb, int64_t k_sh, int64_t k_ss,
                              int64_t v_sb, int64_t v_sh, int64_t v_ss,
                              int64_t o_sb, int64_t o_sh, int64_t o_ss,
                              float softmax_temp, int dtype, void* stream);

/* Band terms of the backward pass of Scatterbrain-local attention (the reference differentiates its op
 * sequence sblocal_attention.py:90-122 with autograd and the backward kernels of
 * fast_transformers.local_product).  For a (query i, key s) pair inside the band, with
 * a = exp(t q_i.k_s - log_norm_i), kb = psi_i.phik_s, df = g_i.v_s - c_i, dm = a df:
 *   key_major = 0 (outer = queries, T rows; inner = keys):  x1 = q, x3 = g, y1 = k, y2 = phik, y3 = v;
 *       o1 = t sum_s dm k_s (T,E), o2 = sum_s df phik_s (T,M); x2, o3 unused (may be NULL)
 *   key_major = 1 (outer = keys, S rows; inner = queries):  x1 = k, x2 = phik, x3 = v, y1 = q, y2 = psi,
 *       y3 = g;  o1 = t sum_i dm q_i (S,E), o2 = sum_i df psi_i (S,M), o3 = sum_i (a - kb) g_i (S,E)
 * All tensors float32, contiguous (BH, rows, width), widths E, M, E; log_norm and c are (BH, T);
 * key_lengths (BH / H) int64 or NULL; (E, M) in {(32,32),(32,64),(64,32),(64,64),(64,128)}. */
int flyhip_sblocal_bwd_band(const float* x1, const float* x2, const float* x3,
                            const float* y1, const float* y2, const float* y3,
                            const float* log_norm, const float* c, const int64_t* key_lengths,
                            float* o1, float* o2, float* o3,
                            int BH, int H, int T, int S, int E, int M, int local_context,
                            float softmax_temp, int key_major, void* stream);

/* flyhip_sblocal_bwd_band for a forward that dropped exact weights with (dropout_p, dropout_seed) (the dropout of
 * sblocal_attention.py:119 / local_attention.py:91, whose mask autograd keeps; here it is formed again from the seed,
 * the hash of flyhip_sblocal_forward): with m = 0 on dropped pairs and 1 / (1 - dropout_p) on kept ones,
 * dm = a (m g_i.v_s - c_i) and o3 = sum_i (m a - kb) g_i; df and o2 are unchanged (the low-rank part is not dropped).
 * dropout_p = 0 is flyhip_sblocal_bwd_band. */
int flyhip_sblocal_bwd_band_dropout(const float* x1, const float* x2, const float* x3,
                                    const float* y1, const float* y2, const float* y3,
                                    const float* log_norm, const float* c, const int64_t* key_lengths,
                                    float* o1, float* o2, float* o3,
                                    int BH, int H, int T, int S, int E, int M, int local_context,
                                    float softmax_temp, int key_major, float dropout_p, uint64_t dropout_seed,
                                    void* stream);

/* flyhip_sblocal_bwd_band_dropout for a forward with an additive attn_mask (flyhip_local_fwd_masked; the reference
 * takes these gradients from autograd through src/models/attention/local_attention.py:68-92): the pair weight is
 * exp(t (q.k + attn_mask[query][key]) - log_norm[query]), and 1 / local_context where log_norm[query] is -inf.
 * attn_mask NULL is flyhip_sblocal_bwd_band_dropout. */
int flyhip_sblocal_bwd_band_masked(const float* x1, const float* x2, const float* x3,
                                   const float* y1, const float* y2, const float* y3,
                                   const float* log_norm, const float* c, const int64_t* key_lengths,
                                   const float* attn_mask,
                                   float* o1, float* o2, float* o3,
                                   int BH, int H, int T, int S, int E, int M, int local_context,
                                   float softmax_temp, int key_major, float dropout_p, uint64_t dropout_seed,
                                   void* stream);

/* The whole backward pass after the feature maps, one call per side (same operand roles as
 * flyhip_sblocal_bwd_band, x2 = the outer rows' own features in both passes: psi for key_major = 0,
 * phik for key_major = 1).  The epilogue adds the low-rank weight outside the band ("all keys minus the
 * band") through the per-head reductions gmat (BH,M,E) | gvec (BH,M) -- phik^T v | sum phik for
 * key_major = 0, psi^T g | psi^T c for key_major = 1 -- and the chain rule through the feature map
 * (feature_maps_sb.py:51-82: features f < M/2 are exp(+sqrt(t) p_f.x - ..), f + M/2 their exp(-..)
 * partners; proj (M/2, E) float32):  d1 = gradient of x1 (d query (T,E) resp. d key (S,E)),
 * d3 = d value (S,E), key_major = 1 only. */
int flyhip_sblocal_bwd(const float* x1, const float* x2, const float* x3,
                       const float* y1, const float* y2, const float* y3,
                       const float* log_norm, const float* c, const int64_t* key_lengths,
                       const float* gmat, const float* gvec, const float* proj,
                       float* d1, float* d3,
                       int BH, int H, int T, int S, int E, int M, int local_context,
                       float softmax_temp, int key_major, void* stream);

/* Everything the two band passes of the backward need besides q, k, v and d out, in three launches (the reference
 * gets it from autograd through softmax_kernel, src/models/attention/feature_maps_sb.py:51-82, and the sums of
 * src/models/attention/sblocal_attention.py:76-80).  Inputs packed float32: q, grad_out, out (BH,T,E), k, v
 * (BH,S,E), log_norm (BH,T), proj (M/2,E) with rows >= mh_valid zero, key_lengths (BH / H) int64 or NULL.
 * Outputs: psi (BH,T,M) = Phi(q) exp(kappa - log_norm), phik (BH,S,M) = Phi(k) exp(-kappa), zero at and past the
 * key length, each row [exp(+.) | exp(-.)] in halves of M/2 with features >= mh_valid zero; kappa = the largest
 * log-feature of a valid key of the (batch, head); c (BH,T) = grad_out . out; kv (BH,M,E) = phik^T v,
 * ksum (BH,M) = sum phik, qg (BH,M,E) = psi^T grad_out, qc (BH,M) = psi^T c.
 * q_images, k_images (both or neither; flyhip_sblocal_bwd_image_bytes(BH, rows, E, M) bytes each): per 32 rows of
 * the side one image of (q, grad_out, psi) resp. (k, v, phik) in two bf16 pieces each, the operands of
 * flyhip_sblocal_bwd_pieces; with them the features are rounded to 17 significant bits everywhere (their two
 * pieces are exact), and psi / phik may be NULL.  scratch: flyhip_sblocal_bwd_prep_scratch(BH,T,S,E,M) floats.
 * (E, M) as for flyhip_sblocal_bwd. */
int64_t flyhip_sblocal_bwd_prep_scratch(int BH, int T, int S, int E, int M);
int64_t flyhip_sblocal_bwd_image_bytes(int BH, int rows, int E, int M);
int flyhip_sblocal_bwd_prep(const float* q, const float* k, const float* v, const float* grad_out,
                            const float* out, const float* log_norm, const float* proj,
                            const int64_t* key_lengths,
                            float* psi, float* phik, float* c,
                            float* kv, float* ksum, float* qg, float* qc,
                            void* q_images, void* k_images,
                            float* scratch, int64_t scratch_floats,
                            int BH, int H, int T, int S, int E, int M, int mh_valid,
                            float softmax_temp, void* stream);

/* flyhip_sblocal_bwd on the bf16 matrix pipe: the same sums and epilogue (same gmat | gvec, proj, d1, d3 and
 * key_major), every product from operands in two bf16 pieces with float32 accumulation.  outer_images /
 * inner_images: the images of flyhip_sblocal_bwd_prep of the outer and of the inner side (queries then keys for
 * key_major = 0, keys then queries for key_major = 1); x1 (BH, outer rows, E) float32: the outer rows themselves
 * (q resp. k), c from the same preparation call.  The epilogue's products run on the bf16 matrix pipe as well
 * (gmat, proj and the image's values in three pieces each).
 * part_ws (may be NULL) of part_ws_floats >= flyhip_sblocal_bwd_parts_floats(BH,T,S,E,M,local_context) floats: with
 * it, problems of fewer 64-row tiles than the GPU holds workgroups walk each tile's band in several parts by as many
 * workgroups and finish in a second launch; without it (or when that function returns 0) every tile is one workgroup.
 * dropout_p, dropout_seed: what the forward was called with (0: none) -- the kernel forms the forward's mask again
 * from the seed (ref: the nn.Dropout of src/models/attention/sblocal_attention.py:119 under autograd). */
int64_t flyhip_sblocal_bwd_parts_floats(int BH, int T, int S, int E, int M, int local_context);
int flyhip_sblocal_bwd_pieces(const void* outer_images, const void* inner_images,
                              const float* x1,
                              const float* log_norm, const float* c, const int64_t* key_lengths,
                              const float* gmat, const float* gvec, const float* proj,
                              float* d1, float* d3, float* part_ws, int64_t part_ws_floats,
                              int BH, int H, int T, int S, int E, int M, int local_context,
                              float softmax_temp, int key_major, float dropout_p, uint64_t dropout_seed,
                              void* stream);

/* flyhip_sblocal_bwd_pieces for Scatterbrain attention on a block-sparse support (the reference takes these
 * gradients from autograd through src/models/attention/sbblocksparse_attention.py:161-212): the exact weights live on
 * the nonzero blocks (16 x 16 or 32 x 32) of a layout instead of a band.  tl_ptr (H * ceil(outer rows / 64) + 1),
 * tl_inner, tl_blk (4 per entry): per (head, 64-row outer tile) the 32-row inner tiles that any of its rows meets on
 * the support, and per entry and group of 16 outer rows (16 w .. 16 w + 15 of the tile) a mask: bit 0 = inner rows
 * 0..15, bit 1 = inner rows 16..31 of that tile are on the support for those rows -- the tables of
 * flyhip_sbblocksparse_fwd for key_major = 0 (outer = queries), the same built from the transposed layout for
 * key_major = 1 (outer = keys).  T, S multiples of 16, no key lengths; images, gmat | gvec, c as for
 * flyhip_sblocal_bwd_pieces.
 * Long lists (n_heavy > 0): tl_skip (H * ceil(outer rows / 64) flags) marks the outer tiles the main launch leaves
 * out, tl_heavy (n_heavy indices head * ceil(outer rows / 64) + tile) lists them; they are walked in heavy_parts
 * parts (2..64) by (batch, tile, part) workgroups of a launch of their own and finished by a third; part_ws of at
 * least flyhip_sbblocksparse_bwd_parts_floats(BH / H, n_heavy, heavy_parts, E, M, key_major) floats.
 * dropout_p, dropout_seed: those of the forward (flyhip_sbblocksparse_fwd), as for flyhip_sblocal_bwd_pieces. */
int64_t flyhip_sbblocksparse_bwd_parts_floats(int B, int n_heavy, int heavy_parts, int E, int M, int key_major);
int flyhip_sbblocksparse_bwd_pieces(const void* outer_images, const void* inner_images,
                                    const float* x1, const float* log_norm, const float* c,
                                    const float* gmat, const float* gvec, const float* proj,
                                    float* d1, float* d3,
                                    const int32_t* tl_ptr, const int32_t* tl_inner, const int32_t* tl_blk,
                                    const int32_t* tl_skip, const int32_t* tl_heavy, int n_heavy, int heavy_parts,
                                    float* part_ws, int64_t part_ws_floats,
                                    int BH, int H, int T, int S, int E, int M,
                                    float softmax_temp, int key_major, float dropout_p, uint64_t dropout_seed,
                                    void* stream);

/* Scatterbrain attention on a block-sparse support (ref: src/models/attention/sbblocksparse_attention.py:109-213
 * for need_weights = False, no masks): as flyhip_sblocal_fwd with one part per query tile, but the
 * exact part covers the nonzero blocks of a layout (16 x 16 or 32 x 32) instead of a band.  Key-side inputs (kfeat,
 * chunk_scale, kv, ksum, kmax) from flyhip_sb_kv_reduce; vt = the tile images that pass leaves when asked for them
 * (then kfeat holds feature images and the band kernel runs on bf16 pieces: head dims up to 64, up to 128
 * features), or NULL (fp32 features in kfeat, the kernel on the fp32 matrix pipe).  tl_ptr (H * ceil(T/64) + 1), tl_inner, tl_mask (4 per
 * entry): per (head, 64-query tile) the 32-key tiles that any of its queries sees on the support, and per entry and
 * group of 16 queries (16 w .. 16 w + 15 of the tile) a mask: bit 0 = keys 0..15, bit 1 = keys 16..31 of that tile
 * are on the support for those queries (32 x 32 blocks: 0 or 3, the same for w = 0, 1 and for w = 2, 3).
 * tl_order (H * ceil(T/64), may be NULL): per
 * head a permutation of its query tiles, the order in which they are started -- longest list first keeps a
 * block-row of global tokens from becoming the tail of the launch.
 * Long lists (n_heavy > 0): tl_heavy (n_heavy entries head * ceil(T/64) + tile) names query tiles whose lists are
 * walked in heavy_parts parts (2..64) by the first workgroups of the launch and finished by a merge launch; those
 * tiles carry the entry -1 - tile in tl_order so that no workgroup takes them whole, and every block-row of such
 * a tile must have at least one block.  Scratch for them: part_ws of B*n_heavy*heavy_parts*64*(D+5) floats and qfeat of
 * B*n_heavy*64*m floats (both NULL when n_heavy == 0).  float32 arithmetic only; T, S multiples of 16.  With the tile
 * images (vt) q, k, v and out may be bfloat16 or float16 tensors: dtype = 0 | (1 << 8) resp. 0 | (2 << 8), here and in the
 * flyhip_sb_kv_reduce call that precedes it -- the kernels widen what they load and round what they store.
 * dropout_p in [0, 1), dropout_seed: the dropout of the exact weights of sbblocksparse_attention.py:200 (the low-rank
 * part and the normaliser see none), by the hash mask that flyhip_sblocal_forward documents;
 * flyhip_sbblocksparse_bwd_pieces takes the same two values and forms the mask again. */
int flyhip_sbblocksparse_fwd(const void* q, const void* k, const void* v, const float* proj,
                             const void* kfeat, const void* vt, const float* chunk_scale,
                             const float* kv, const float* ksum, const float* kmax,
                             const int32_t* tl_ptr, const int32_t* tl_inner, const int32_t* tl_mask,
                             const int32_t* tl_order, const int32_t* tl_heavy, int n_heavy, int heavy_parts,
                             float* part_ws, float* qfeat,
                             void* out, float* log_norm,
                             int B, int H, int T, int S, int E, int D, int mh, int mh_valid,
                             int64_t q_sb, int64_t q_sh, int64_t q_ss,
                             int64_t k_sb, int64_t k_sh, int64_t k_ss,
                             int64_t v_sb, int64_t v_sh, int64_t v_ss,
                             int64_t o_sb, int64_t o_sh, int64_t o_ss,
                             float softmax_temp, int dtype, float dropout_p, uint64_t dropout_seed, void* stream);

/* Plain local attention, no random features (ref: src/models/attention/local_attention.py:68-92;
 * fast_transformers.local_product): out[i] = softmax over the band -(lc/2) <= s - i < (lc+1)/2, s below
 * the key length, of t q_i.k_s, times v.  q (B,T,H,E), k (B,S,H,E), v (B,S,H,D), out (B,T,H,D) via
 * (batch, head, seq) strides, innermost contiguous; E = D in {32,64,128}; key_lengths (B) int64 or
 * NULL.  A query with no valid key gets a zero row (local_attention.py:74-84).
 * dtype: float32 (both products on the fp32 matrix pipe), bfloat16 or float16 (both on the 16x16x32 MFMA of the
 * type, the weights rounded to it for the second product; float16 needs strides in multiples of 8 elements and
 * 16-byte aligned pointers, bfloat16 with other strides runs on the fp32 pipe). */
int flyhip_local_fwd(const void* q, const void* k, const void* v, const int64_t* key_lengths, void* out,
                     int B, int H, int T, int S, int E, int D, int local_context,
                     int64_t q_sb, int64_t q_sh, int64_t q_ss,
                     int64_t k_sb, int64_t k_sh, int64_t k_ss,
                     int64_t v_sb, int64_t v_sh, int64_t v_ss,
                     int64_t o_sb, int64_t o_sh, int64_t o_ss,
                     float softmax_temp, int dtype, void* stream);

/* flyhip_local_fwd that also writes, when lse is not NULL, the log of every query's softmax
 * denominator (B,H,T) float32 -- what the backward pass needs to evaluate the weights again (the
 * reference keeps the whole (B,H,T,local_context) weight tensor for autograd, local_attention.py:75-91);
 * 0 for a query without keys. */
int flyhip_local_fwd_lse(const void* q, const void* k, const void* v, const int64_t* key_lengths, void* out,
                         float* lse,
                         int B, int H, int T, int S, int E, int D, int local_context,
                         int64_t q_sb, int64_t q_sh, int64_t q_ss,
                         int64_t k_sb, int64_t k_sh, int64_t k_ss,
                         int64_t v_sb, int64_t v_sh, int64_t v_ss,
                         int64_t o_sb, int64_t o_sh, int64_t o_ss,
                         float softmax_temp, int dtype, void* stream);

/* flyhip_local_fwd_lse with the dropout of LocalAttention.forward (ref: src/models/attention/local_attention.py:91,
 * `self.dropout(torch.softmax(...))`): every weight is dropped with probability dropout_p in [0, 1) after the softmax
 * (lse is that of the undropped softmax) and the kept ones are scaled by 1 / (1 - dropout_p).  The mask is the hash
 * of (seed, (b H + h) T + query, key) that flyhip_sblocal_forward documents; flyhip_sblocal_bwd_band_dropout forms
 * it again.  dropout_p = 0 is flyhip_local_fwd_lse. */
int flyhip_local_fwd_dropout(const void* q, const void* k, const void* v, const int64_t* key_lengths, void* out,
                             float* lse,
                             int B, int H, int T, int S, int E, int D, int local_context,
                             int64_t q_sb, int64_t q_sh, int64_t q_ss,
                             int64_t k_sb, int64_t k_sh, int64_t k_ss,
                             int64_t v_sb, int64_t v_sh, int64_t v_ss,
                             int64_t o_sb, int64_t o_sh, int64_t o_ss,
                             float softmax_temp, int dtype, float dropout_p, uint64_t dropout_seed, void* stream);

/* flyhip_local_fwd_dropout with the attn_mask of LocalAttention.forward (ref: src/models/attention/local_attention.py:
 * 53-56, 68-81): attn_mask (T, S) float32, rows contiguous, or NULL -- the mask's additive_matrix_finite (0 / -1e24; any
 * finite bias is allowed), added to q.k before the temperature.  -1e24 absorbs the product in float32, so a query
 * whose visible keys are all masked weighs every position of its band 1 / local_context, those outside the keys
 * included (they add nothing to the output), as the reference's softmax over the packed band does; its lse entry is
 * -inf, which flyhip_sblocal_bwd_band_masked reads as that case. */
int flyhip_local_fwd_masked(const void* q, const void* k, const void* v, const int64_t* key_lengths,
                            const float* attn_mask, void* out, float* lse,
                            int B, int H, int T, int S, int E, int D, int local_context,
                            int64_t q_sb, int64_t q_sh, int64_t q_ss,
                            int64_t k_sb, int64_t k_sh, int64_t k_ss,
                            int64_t v_sb, int64_t v_sh, int64_t v_ss,
                            int64_t o_sb, int64_t o_sh, int64_t o_ss,
                            float softmax_temp, int dtype, float dropout_p, uint64_t dropout_seed, void* stream);

/* Gradients of flyhip_local_fwd for bfloat16 or float16 tensors (the reference takes them from autograd through
 * fast_transformers.local_product, src/models/attention/local_attention.py:68-92): with P = the band softmax formed again
 * as exp(t q.k - lse), g = grad_out and delta[b][h][i] = g_i . out_i (float32 (B,H,T) like lse: caller-owned scratch
 * that the first launch fills from out, the forward's output, and the second reads):
 * dv_s = sum_i P_is g_i, dS_is = P_is (g_i.v_s - delta_i), dq_i = t sum_s dS_is k_s, dk_s = t sum_i dS_is q_i.  Two
 * launches (query-major for dq, key-major for dk and dv) on the 16x16x32 MFMA of the input type, P and dS rounded to it.
 * q, out, grad_out, dq (B,T,H,E) and k, v, dk, dv (B,S,H,E) via (batch, head, seq) strides in elements, innermost
 * contiguous, E in {32,64,128}; input strides in multiples of 8 elements and 16-byte aligned pointers, output strides in
 * multiples of 4.  Every row of dq, dk, dv is written (zeros where a row has no pair in the band).  No attn_mask, no
 * dropout: those gradients run on flyhip_sblocal_bwd_band_masked. */
int flyhip_local_bwd(const void* q, const void* k, const void* v, const void* out, const void* grad_out,
                     const float* lse, const int64_t* key_lengths, float* delta,
                     void* dq, void* dk, void* dv,
                     int B, int H, int T, int S, int E, int local_context,
                     int64_t q_sb, int64_t q_sh, int64_t q_ss,
                     int64_t k_sb, int64_t k_sh, int64_t k_ss,
                     int64_t v_sb, int64_t v_sh, int64_t v_ss,
                     int64_t o_sb, int64_t o_sh, int64_t o_ss,
                     int64_t g_sb, int64_t g_sh, int64_t g_ss,
                     int64_t dq_sb, int64_t dq_sh, int64_t dq_ss,
                     int64_t dk_sb, int64_t dk_sh, int64_t dk_ss,
                     int64_t dv_sb, int64_t dv_sh, int64_t dv_ss,
                     float softmax_temp, int dtype, void* stream);

/* Measurement hook (no counterpart in the reference): the two caller-owned hipEvent_t receive the begin
 * and the end time stamp of the fused band kernel's launch (hipExtLaunchKernelGGL) in the NEXT
 * flyhip_sblocal_fwd call of the calling thread, on its stream, and are then forgotten: their elapsed time
 * is the kernel's duration.  Pass NULLs to clear. */
int flyhip_sb_time_next_fwd(void* event_before, void* event_after);

/* ------------------------------------------------------------------------------------------
 * Block-sparse matmuls (ref: src/models/attention/blocksparse_matmul.py; matmul.__call__ :656,
 * _sdd_matmul :279-346, _dds_matmul :444-488, _dsd_matmul :491-535).
 * Sparse tensors are (Z, nnz, blk, blk); block n is the n-th nonzero of the (H, rows, cols)
 * layout in row-major order (ref: blocksparse_utils.py:8-19).  blk in {16,32,64,128}.
 * ---------------------------------------------------------------------------------------- */

/* SDD: c[z, n] = A[z, h_n, rows of block-row i_n, :] . B[z, h_n, rows of block-col j_n, :]^T where
 * A(m,k) / B(n,k) are addressed with (batch, head, row, k) strides (this covers trans_a/trans_b).
 * lut: int32 (nnz,4) rows (head, block_row, block_col, block_id) (ref: make_sdd_lut :261-276).
 * row_ptr / row_blk / row_col (optional, may be NULL): the same blocks grouped per (head, block-row),
 * n_brow = H * rows/blk of them; with these, 32x32 blocks of a 2-byte type take a faster kernel that
 * keeps the A tile of a block-row in registers.
 * uni_ptr / uni_inner / uni_blk (optional, may be NULL; used with the row tables): for every group of
 * four consecutive block-rows of a head (ceil(rows/4) groups per head, head-major), the union of
 * the rows' block-columns in increasing order: uni_ptr int32 (n_groups+1), uni_inner int32 (n_union)
 * the block-column, uni_blk int32 (n_union,4) the block id of (row 4g+w, that column) or -1.  With
 * them the four rows share every B tile through LDS; worth passing when neighbouring rows have
 * most columns in common. */
int flyhip_bs_sdd(const void* a, const void* b, void* c, const int32_t* lut, int nnz,
                  const int32_t* row_ptr, const int32_t* row_blk, const int32_t* row_col,
                  int n_brow, int brows_per_head,
                  const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                  int Z, int K, int blk,
                  int64_t a_sz, int64_t a_sh, int64_t a_sm, int64_t a_sk,
                  int64_t b_sz, int64_t b_sh, int64_t b_sn, int64_t b_sk,
                  int dtype, void* stream);

/* Score gradient of a block-sparse attention core in one kernel: ds[z, n] = scale * p[z, n] * (dout[rows of
 * block-row i_n] . v[rows of block-col j_n]^T - delta[row]), i.e. the sdd that forms dP = dO V^T fused with
 * the backward of softmax(scale * s) (ref: the autograd chain behind blocksparse_attention.py:134-160:
 * _sdd_matmul :279-346 followed by the softmax backward).  p, ds (Z, nnz, 32, 32) of bf16 / fp16;
 * dout (Z,H,rows,K), v (Z,H,cols,K) with (batch, head, row) strides and contiguous K in {32,..,128};
 * delta fp32 (Z, H, rows) = rowsum(dout * out); uni_* the union table of flyhip_bs_sdd (required). */
int flyhip_bs_sdd_dsoftmax(const void* dout, const void* v, const void* p, const float* delta, void* ds,
                           const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                           int nnz, int n_heads, int brows_per_head, int Z, int K, int blk,
                           int64_t a_sz, int64_t a_sh, int64_t a_sm,
                           int64_t b_sz, int64_t b_sh, int64_t b_sn,
                           float scale, int dtype, void* stream);

/* SDD with the contraction index slowest in both operands: c32[z, n] += A[z, h_n, :, block-row i_n]^T .
 * B[z, h_n, :, block-col j_n], A (Z,H,K,M) and B (Z,H,K,N) with (batch, head, k) strides and contiguous
 * features -- the weight gradient x^T dy of a block-sparse linear layer, K = tokens (ref: the 'sdd'
 * call of the backward pass, blocksparse_matmul.py:562-587 -> _sdd_matmul :279-346).  32x32 blocks
 * of bf16 / fp16.  c32 is fp32 (Z, nnz, 32, 32), ZEROED by the caller: slices of k_slice tokens
 * (a multiple of 32) are accumulated into it with float atomics; the caller rounds it to the
 * output type.  row_ptr / row_blk / row_col as in flyhip_bs_sdd; grp_row0 / grp_n: groups of at most
 * four consecutive block-rows of a head with identical column lists (every block-row in exactly one
 * group); max_row_nnz = the longest column list. */
int flyhip_bs_sdd_kmajor(const void* a, const void* b, float* c32,
                         const int32_t* row_ptr, const int32_t* row_blk, const int32_t* row_col,
                         const int32_t* grp_row0, const int32_t* grp_n, int n_grp, int max_row_nnz,
                         int brows_per_head, int nnz, int Z, int K, int k_slice, int blk,
                         int64_t a_sz, int64_t a_sh, int64_t a_sk,
                         int64_t b_sz, int64_t b_sh, int64_t b_sk,
                         int dtype, void* stream);

/* DSD: c (Z,H,M,N) = op(sparse a) . dense b.  Segment s = (head, output block-row); seg_ptr
 * (n_seg+1), seg_blk (block id), seg_inner (inner block index) int32 list the blocks reduced into
 * it; n_seg = H * M/blk; an empty segment writes zeros (ref: make_dxx_lut :356-441 plays this
 * role).  trans_a != 0 reads every sparse block transposed.  b(k,n) and c(m,n) via strides.
 * uni_ptr / uni_inner / uni_blk (optional, may be NULL; trans_a == 0 only): the union table of
 * flyhip_bs_sdd over groups of four output block-rows; with it the four rows share every tile of
 * b through LDS. */
int flyhip_bs_dsd(const void* a_sp, const void* b, void* c,
                  const int32_t* seg_ptr, const int32_t* seg_blk, const int32_t* seg_inner,
                  const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                  int n_seg, int rows_per_head, int Z, int N, int blk, int trans_a,
                  int64_t a_sz,
                  int64_t b_sz, int64_t b_sh, int64_t b_sk, int64_t b_sn,
                  int64_t c_sz, int64_t c_sh, int64_t c_sm, int64_t c_sn,
                  int dtype, void* stream);

/* DDS: c (Z,H,M,N) = dense a . op(sparse b).  Segment s = (head, output block-column); trans_b != 0
 * reads every sparse block transposed (the BlockSparseLinear case, ref:
 * src/models/layers/blocksparse_linear.py:119-120,152-162).  a(m,k) and c(m,n) via strides.
 * grp_row0 / grp_n (optional, may be NULL, n_grp entries): groups of at most four consecutive segments
 * of one head whose reduction lists visit the same inner blocks in the same order (first segment
 * and count per group, covering every segment once; max_seg_len = longest reduction list); with them, 32x32 blocks of a 2-byte type with
 * trans_b take a tiled kernel that treats each group as a small dense GEMM. */
int flyhip_bs_dds(const void* a, const void* b_sp, void* c,
                  const int32_t* seg_ptr, const int32_t* seg_blk, const int32_t* seg_inner,
                  const int32_t* grp_row0, const int32_t* grp_n, int n_grp, int max_seg_len,
                  int n_seg, int cols_per_head, int Z, int M, int blk, int trans_b,
                  int64_t a_sz, int64_t a_sh, int64_t a_sm, int64_t a_sk,
                  int64_t b_sz,
                  int64_t c_sz, int64_t c_sh, int64_t c_sm, int64_t c_sn,
                  int dtype, void* stream);

/* Fused block-sparse attention: out = softmax(scale * q k^T + key mask) v over the nonzero blocks of
 * the layout, in one pass -- the SDD -> block softmax -> DSD sequence of BlockSparseAttention.forward
 * (ref: src/models/attention/blocksparse_attention.py:134-160) without the (Z, nnz, blk, blk) score
 * and probability tensors.  32x32 blocks of bf16 / fp16 only; q (Z,H,rows,D), k / v (Z,H,cols,D),
 * out (Z,H,rows,D) via (batch, head, row) strides with D contiguous, D in {32,64,128};
 * rows = 32 * brows_per_head.  uni_ptr / uni_inner / uni_blk: the union table described at
 * flyhip_bs_sdd built for groups of rows_per_group (4 or 8) consecutive block-rows (uni_blk is
 * (n_union, rows_per_group); only its sign is used).  key_mask (optional, may be NULL): fp32
 * (Z, cols) additive term per key (0 or -inf: the additive form of key_padding_mask,
 * blocksparse_attention.py:148-150), row stride key_mask_stride.  A query whose keys are all
 * masked, or whose block-row is empty, gets a zero row (the reference's nan_to_num_, :156-158). */
int flyhip_bs_attn(const void* q, const void* k, const void* v, void* out,
                   const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                   int rows_per_group, const float* key_mask, int64_t key_mask_stride,
                   int Z, int H, int brows_per_head, int D, int blk,
                   int64_t q_sz, int64_t q_sh, int64_t q_sm,
                   int64_t k_sz, int64_t k_sh, int64_t k_sn,
                   int64_t v_sz, int64_t v_sh, int64_t v_sn,
                   int64_t o_sz, int64_t o_sh, int64_t o_sm,
                   float scale, int dtype, void* stream);

/* flyhip_bs_attn that also writes, when lse2 is not NULL, the base-2 logarithm of every row's softmax
 * denominator, (Z, H, 32 * brows_per_head) float32, +inf for a row without a finite score: all a
 * backward pass needs to form the probabilities again (the reference keeps the (Z, nnz, 32, 32)
 * probability tensor for autograd, blocksparse_attention.py:146-160). */
int flyhip_bs_attn_lse(const void* q, const void* k, const void* v, void* out, float* lse2,
                       const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                       int rows_per_group, const float* key_mask, int64_t key_mask_stride,
                       int Z, int H, int brows_per_head, int D, int blk,
                       int64_t q_sz, int64_t q_sh, int64_t q_sm,
                       int64_t k_sz, int64_t k_sh, int64_t k_sn,
                       int64_t v_sz, int64_t v_sh, int64_t v_sn,
                       int64_t o_sz, int64_t o_sh, int64_t o_sm,
                       float scale, int dtype, void* stream);

/* flyhip_bs_attn_lse with the attention mask of BlockSparseAttention.forward as well (ref:
 * src/models/attention/blocksparse_attention.py:124-127,146-152: attn_mask.additive_matrix handed to the block
 * softmax with attn_mask_mode='add'): attn_mask (optional, may be NULL) is fp32 (32 * brows_per_head, cols), row
 * stride attn_mask_stride (a multiple of 4), an additive term per (query, key) shared by every batch entry and head --
 * 0 / -inf from a FullMask, or any finite bias.  Only entries inside nonzero blocks are read.  A query without a
 * finite score gets a zero row (:156-158). */
int flyhip_bs_attn_masks(const void* q, const void* k, const void* v, void* out, float* lse2,
                         const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                         int rows_per_group, const float* key_mask, int64_t key_mask_stride,
                         const float* attn_mask, int64_t attn_mask_stride,
                         int Z, int H, int brows_per_head, int D, int blk,
                         int64_t q_sz, int64_t q_sh, int64_t q_sm,
                         int64_t k_sz, int64_t k_sh, int64_t k_sn,
                         int64_t v_sz, int64_t v_sh, int64_t v_sn,
                         int64_t o_sz, int64_t o_sh, int64_t o_sm,
                         float scale, int dtype, void* stream);

/* Gradients of flyhip_bs_attn_lse (the one-kernel block-sparse attention without masks; the reference takes them from
 * autograd through sdd, softmax and dsd, src/models/attention/blocksparse_attention.py:134-160) without the
 * probabilities in memory: with P = 2^(scale log2e q.k - lse2[query]) on the nonzero 32 x 32 blocks, g = grad_out and
 * delta = rowsum(g * out): dv = P^T g, dS = P (g v^T - delta), dq = scale dS k, dk = scale dS^T q.  Two launches on
 * the 16x16x32 MFMA of the input type: query-major over groups of four block-rows (dq; fills delta, caller-owned
 * float32 scratch shaped like lse2) and key-major over groups of four block-columns (dk, dv).  row_* = union_table of
 * the layout, col_* = the same of the transposed layout (block ids are only tested for >= 0).  q, out, grad_out, dq
 * (Z, H, 32 brows, E) and k, v, dk, dv (Z, H, 32 bcols, E) via (batch, head, row) strides in elements, E in {32, 64},
 * bfloat16 or float16; input strides in multiples of 8 and 16-byte aligned pointers, output strides in multiples of 4.
 * dropout_p, dropout_seed: those of a flyhip_bs_attn_dropout forward (0 for none): the mask is formed again from the
 * hash of (seed, (z H + head) L + query, key); dv takes m P and dS = P (m g.v - delta), m = 0 or 1 / (1 - p).
 * key_mask (Z, keys) and attn_mask (queries, keys), both optional: the additive masks of a flyhip_bs_attn_masks forward
 * (float32, row strides in multiples of 4), added to scale q.k before the exponential; not together with dropout. */
int flyhip_bs_attn_bwd(const void* q, const void* k, const void* v, const void* out, const void* grad_out,
                       const float* lse2, float* delta, void* dq, void* dk, void* dv,
                       const int32_t* row_ptr, const int32_t* row_inner, const int32_t* row_blk,
                       const int32_t* col_ptr, const int32_t* col_inner, const int32_t* col_blk,
                       int n_heads, int brows_per_head, int bcols_per_head, int Z, int E,
                       int64_t q_sz, int64_t q_sh, int64_t q_sm, int64_t k_sz, int64_t k_sh, int64_t k_sm,
                       int64_t v_sz, int64_t v_sh, int64_t v_sm, int64_t o_sz, int64_t o_sh, int64_t o_sm,
                       int64_t g_sz, int64_t g_sh, int64_t g_sm,
                       int64_t dq_sz, int64_t dq_sh, int64_t dq_sm, int64_t dk_sz, int64_t dk_sh, int64_t dk_sm,
                       int64_t dv_sz, int64_t dv_sh, int64_t dv_sm,
                       float scale, int dtype, float dropout_p, uint64_t dropout_seed,
                       const float* key_mask, int64_t key_mask_stride, const float* attn_mask, int64_t attn_mask_stride,
                       void* stream);

/* flyhip_bs_attn_masks with the dropout of BlockSparseAttention.forward (ref:
 * src/models/attention/blocksparse_attention.py:160, `dsd_nn(self.dropout(attn), v)`; the constructor's default
 * attention_dropout is 0.1, :31): every probability is dropped with probability dropout_p in [0, 1) after the softmax
 * (the denominator sums all of them) and the kept ones are scaled by 1 / (1 - dropout_p).  No mask tensor exists:
 * keys 2c and 2c + 1 of (batch z, head h, query i) share the 32-bit hash mix(mix(((z H + h) L + i) * 0x9E3779B1 + s)
 * + c * 0x632BE5AB) -- L = 32 * brows_per_head, mix = the 32-bit finaliser of MurmurHash3, s = the 64-bit seed folded
 * to 32 bits (low ^ high * 0x9E3779B1) -- key 2c takes its low and key 2c + 1 its high 16 bits, and a probability is
 * kept iff its half >= floor(dropout_p 2^16); flyhip_bs_sdd_prob_dsoftmax_dropout forms the same mask again.
 * lse2 is that of the undropped softmax.  dropout_p = 0 is flyhip_bs_attn_masks. */
int flyhip_bs_attn_dropout(const void* q, const void* k, const void* v, void* out, float* lse2,
                           const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                           int rows_per_group, const float* key_mask, int64_t key_mask_stride,
                           const float* attn_mask, int64_t attn_mask_stride,
                           int Z, int H, int brows_per_head, int D, int blk,
                           int64_t q_sz, int64_t q_sh, int64_t q_sm,
                           int64_t k_sz, int64_t k_sh, int64_t k_sn,
                           int64_t v_sz, int64_t v_sh, int64_t v_sn,
                           int64_t o_sz, int64_t o_sh, int64_t o_sm,
                           float scale, int dtype, float dropout_p, uint64_t dropout_seed, void* stream);

/* The probabilities of that attention again, in the block-sparse format: p = exp(scale * q k^T - lse) on
 * the nonzero blocks, as one sdd (blocksparse_matmul.py:279-346) with an exponential epilogue;
 * lse2 as written by flyhip_bs_attn_lse; tables as for flyhip_bs_sdd's shared-tile path (four
 * block-rows per group). */
int flyhip_bs_sdd_prob(const void* q, const void* k, const float* lse2, void* p,
                       const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                       int nnz, int n_heads, int brows_per_head, int Z, int K, int blk,
                       int64_t a_sz, int64_t a_sh, int64_t a_sm,
                       int64_t b_sz, int64_t b_sh, int64_t b_sn,
                       float scale, int dtype, void* stream);

/* flyhip_bs_sdd_prob and flyhip_bs_sdd_dsoftmax in one pass over the nonzero blocks: both products
 * (q k^T and d out v^T) per block, p = exp(scale q k^T - lse) written to p and
 * ds = scale * p * (d out v^T - delta[row]) to ds, both (Z, nnz, 32, 32); neither the scores nor
 * d p exist in memory (the reference's autograd chain through blocksparse_attention.py:134-160
 * materialises both).  The gradient of q comes out of the same pass: dq = ds k over the row's blocks
 * (Z, H, rows, K) through (batch, head, row) strides.  delta (Z, H, rows) float32 = rowsum(d out * out)
 * may be NULL when out (the forward's result, strided like d out) is given: it is then formed here. */
int flyhip_bs_sdd_prob_dsoftmax(const void* dout, const void* v, const void* q, const void* k,
                                const float* delta, const void* out, const float* lse2, void* ds, void* p, void* dq,
                                const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                                int nnz, int n_heads, int brows_per_head, int Z, int K, int blk,
                                int64_t do_sz, int64_t do_sh, int64_t do_sm,
                                int64_t v_sz, int64_t v_sh, int64_t v_sn,
                                int64_t q_sz, int64_t q_sh, int64_t q_sm,
                                int64_t k_sz, int64_t k_sh, int64_t k_sn,
                                int64_t dq_sz, int64_t dq_sh, int64_t dq_sm,
                                int64_t o_sz, int64_t o_sh, int64_t o_sm,
                                float scale, int dtype, void* stream);

/* flyhip_bs_sdd_prob_dsoftmax for a forward that dropped probabilities (flyhip_bs_attn_dropout with the same
 * dropout_p, dropout_seed and shapes): with m = 0 on dropped pairs and 1 / (1 - dropout_p) on kept ones, p receives
 * m * p -- the operand of dv = (m p)^T d out -- and ds = scale * p * (m * d out v^T - delta[row]); delta =
 * rowsum(d out * out) as before (out being the dropped forward's result).  The chain is the one autograd builds
 * through blocksparse_attention.py:146-160 with nn.Dropout's mask kept. */
int flyhip_bs_sdd_prob_dsoftmax_dropout(const void* dout, const void* v, const void* q, const void* k,
                                const float* delta, const void* out, const float* lse2, void* ds, void* p, void* dq,
                                const int32_t* uni_ptr, const int32_t* uni_inner, const int32_t* uni_blk,
                                int nnz, int n_heads, int brows_per_head, int Z, int K, int blk,
                                int64_t do_sz, int64_t do_sh, int64_t do_sm,
                                int64_t v_sz, int64_t v_sh, int64_t v_sn,
                                int64_t q_sz, int64_t q_sh, int64_t q_sm,
                                int64_t k_sz, int64_t k_sh, int64_t k_sn,
                                int64_t dq_sz, int64_t dq_sh, int64_t dq_sm,
                                int64_t o_sz, int64_t o_sh, int64_t o_sm,
                                float scale, int dtype, float dropout_p, uint64_t dropout_seed, void* stream);

/* ------------------------------------------------------------------------------------------
 * Block-sparse row operations.  row_ptr (n_brow+1) / row_blk / row_col int32: for every
 * (head, block-row) the ids and block-columns of its nonzero blocks (the information of the
 * reference's row LUT, ref: blocksparse_logsumexp.py:107-128).  n_brow = H * M/blk.
 * ---------------------------------------------------------------------------------------- */

/* In-place softmax over the nonzero blocks of each row of x*scale + kpm[z,col] + am[row,col]
 * (ref: triton.ops.blocksparse.softmax as called at blocksparse_attention.py:146-152).
 * kpm (Z, kpm_stride) / am (rows, am_stride) fp32 additive or NULL; *_mul != 0 selects the
 * 'mul' mode (0 -> -inf, nonzero -> 0).  A row with no finite entry becomes NaN.  max_row_nnz = the
 * largest number of blocks in any block-row (an upper bound is fine). */
int flyhip_bs_softmax(void* x, const int32_t* row_ptr, const int32_t* row_blk, const int32_t* row_col,
                      int n_brow, int brows_per_head, int max_row_nnz, int Z, int blk, int64_t x_sz, float scale,
                      const float* kpm, int64_t kpm_stride, int kpm_mul,
                      const float* am, int64_t am_stride, int am_mul,
                      int dtype, void* stream);

/* Backward of flyhip_bs_softmax without masks in the gradient: dx = scale * y * (dy - rowsum(dy * y)) over
 * the nonzero blocks, y the softmax output (ref: the backward of triton.ops.blocksparse.softmax,
 * reached from blocksparse_attention.py:146-152 under autograd).  32x32 blocks of bf16 / fp16, at most
 * 64 blocks per block-row; y, dy, dx (Z, nnz, 32, 32) contiguous per batch, batch stride y_sz. */
int flyhip_bs_softmax_bwd(const void* y, const void* dy, void* dx,
                          const int32_t* row_ptr, const int32_t* row_blk,
                          int n_brow, int max_row_nnz, int Z, int blk, int64_t y_sz,
                          float scale, int dtype, void* stream);

/* Row reduction over nonzero blocks -> out (Z, n_brow*blk) in x's dtype: op 0 = logsumexp
 * (ref: blocksparse_logsumexp.py:161-184), op 1 = sum (ref: blocksparse_sum.py:156-179).
 * Rows of an empty block-row give 0. */
int flyhip_bs_rowreduce(const void* x, void* out, const int32_t* row_ptr, const int32_t* row_blk,
                        int n_brow, int Z, int blk, int64_t x_sz, int op, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif
