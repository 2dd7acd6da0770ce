/* veloxquant_hip.h -- C ABI of the MI355X (gfx950) KV-cache compression library.
 *
 * One shared library (libveloxquant_hip.so) replaces the Metal kernel layer of
 * VeloxQuant-MLX for the KIVI / VecInfer hot path.  Every entry point
 *   - takes plain device pointers and sizes (no framework types),
 *   - enqueues work on the HIP stream it is given and returns without syncing,
 *   - never allocates or frees device memory and keeps no pointer after return,
 *   - returns 0 on success or a negative VQ_ERR_* code; vq_last_error() holds
 *     the message of the calling thread's last failure.
 * Citations name the reference interface each entry point stands in for
 * (paths relative to the VeloxQuant-MLX source tree).
 */
#ifndef VELOXQUANT_HIP_H
#define VELOXQUANT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types */
enum { VQ_F16 = 0, VQ_BF16 = 1, VQ_F32 = 2, VQ_U8 = 3, VQ_I32 = 4, VQ_U32 = 5 };

/* status codes */
enum {
    VQ_OK = 0,
    VQ_ERR_INVALID = -1,     /* bad shape / dtype / range (maps to ValueError)   */
    VQ_ERR_UNSUPPORTED = -2, /* valid request outside what the kernels cover     */
    VQ_ERR_WORKSPACE = -3,   /* workspace missing or too small                   */
    VQ_ERR_HIP = -4          /* a HIP runtime call failed                        */
};

/* axis of group quantisation inside the trailing [S, D] dims */
enum { VQ_AXIS_TOKEN = 0 /* keys: groups run along S (python axis -2)     */,
       VQ_AXIS_CHANNEL = 1 /* values: groups run along D (python axis -1) */ };

/* layout of packed VALUE codes and their scale/zero:
 *   VQ_V_CHANNEL_PACKED  words hold consecutive channels of one token:
 *                        codes [BH, S, ceil(D/per)], scale/zero [BH, S, GV]
 *                        (the image _pack_indices gives for [.., S, D] codes)
 *   VQ_V_TOKEN_PACKED    words hold consecutive tokens of one channel:
 *                        codes [BH, ceil(S/per), D], scale/zero [BH, GV, S]
 *                        (_pack_indices applied to the [.., D, S] transpose and
 *                        stored with the word axis ahead of D); this is the
 *                        layout the MFMA decode kernel streams
 * per = 32 / pack_bits. */
enum { VQ_V_CHANNEL_PACKED = 0, VQ_V_TOKEN_PACKED = 1 };

int vq_abi_version(void);
/* copies the calling thread's last error text; returns its length */
int vq_last_error(char *buf, size_t n);
/* number of HIP devices visible, or a negative VQ_ERR_HIP */
int vq_device_count(void);

/* ---- KIVI group quantisation -------------------------------------------- */

/* Fused quantise -> dequantise round trip, out = cast(code*scale + min).
 * Replaces kivi_group_quant_dequant(x, axis, group_size, levels, eps)
 * (veloxquant_mlx/metal/_kivi_quant.py:138-207) and the pure-MLX
 * KIVIKVCache._quant_dequant_along (veloxquant_mlx/cache/kivi_cache.py:151-201).
 * x/out: [BH, S, D] contiguous, same dtype (VQ_F16 / VQ_BF16 / VQ_F32). */
int vq_kivi_quant_dequant(const void *x, void *out, int dtype, int64_t BH, int64_t S, int64_t D,
                          int axis, int group, int levels, float eps, void *stream);

/* The same round trip along the token axis with a level count per channel: channel c of slab bh has
 * levels_hi levels where hi_mask[bh * D + c] != 0 and levels_lo otherwise.  One launch for
 * quantize_mixed_channels (veloxquant_mlx/quantizers/kitty.py:138-169), which forms the hi-bit and the
 * lo-bit reconstruction of the whole tensor and selects per channel.  head_dim 128, groups of 32 or 64
 * tokens; x/out [BH, S, 128] contiguous and 16-byte aligned, hi_mask [BH, 128] bytes, 8-byte aligned. */
int vq_kivi_quant_dequant_mixed(const void *x, void *out, int dtype, int64_t BH, int64_t S, int64_t D, int group,
                                int levels_lo, int levels_hi, const uint8_t *hi_mask, float eps, void *stream);

/* The same round trip along the token axis with a level count per token group: group_levels (device, float,
 * ceil(S / group) entries, the same for every slab) holds 2^bits - 1 for the group's bit width, or 0 for a group
 * that passes through unchanged.  One launch for age_tier_quantize (veloxquant_mlx/quantizers/age_tiered.py:117-174),
 * which quantises every stretch of windows of one age tier on its own.  head_dim 128, groups of 32 or 64 tokens,
 * fp16 or bf16 rows; x/out [BH, S, 128] contiguous, 16-byte aligned, not aliased. */
int vq_kivi_quant_dequant_grouplevels(const void *x, void *out, int dtype, int64_t BH, int64_t S, int64_t D, int group,
                                      const float *group_levels, float eps, void *stream);

/* Per-channel sums over the tokens of x [N, S, D] (slab stride x_stride_n elements), accumulated in double:
 * partial[((n * chunks + k) * 2 + 0) * D + c] = sum, [... + 1 ...] = sum of squares of channel c over the
 * k-th of `chunks` stretches of tokens; the caller adds the chunks.  The population variance Kitty ranks
 * channels by (mx.var over the float32 copy, veloxquant_mlx/quantizers/kitty.py:44-67,
 * veloxquant_mlx/cache/kitty_cache.py:96-104) in one pass over the stored rows.  head_dim 64 / 128 / 256. */
int vq_channel_moments(const void *x, int dtype, int64_t N, int64_t S, int64_t D, int64_t x_stride_n, double *partial,
                       int chunks, void *stream);

/* variance[n * D + c] = max(sq / S - (sum / S)^2, 0), float32, from the partial sums vq_channel_moments wrote
 * (chunks added in order, double arithmetic): the rest of the same mx.var (veloxquant_mlx/quantizers/kitty.py:44-67,
 * veloxquant_mlx/cache/kitty_cache.py:96-104) in one launch. */
int vq_channel_variance(const double *partial, int64_t N, int chunks, int64_t D, int64_t S, float *variance, void *stream);

/* mask[n * D + c] = 1 where channel c is among the n_hi channels of largest variance[n][:], 0 elsewhere: the rank of
 * a channel is its place in a stable ascending sort of -variance (equal variances: the lower channel first, a NaN
 * after every number), which is the double argsort of veloxquant_mlx/quantizers/kitty.py:112-135.  D <= 1024. */
int vq_channel_hi_mask(const float *variance, int64_t N, int64_t D, int64_t n_hi, uint8_t *mask, void *stream);

/* out[r] = L2 norm of row r of x [n_rows, D], float32 arithmetic (head_dim 64 / 128 / 256).  The salience
 * signal of ZipCacheKVCache (mx.linalg.norm over the channels of the float32 copy,
 * veloxquant_mlx/cache/zipcache_cache.py:176-180) without materialising that copy. */
int vq_row_norms(const void *x, int dtype, int64_t n_rows, int64_t D, float *out, void *stream);

/* Routing order of a salience split: order[bh] = the positions of the S - n_hi rows outside the n_hi largest
 * norms[bh] (non-negative float32, [BH, S]) in ascending order, then the positions of the n_hi largest in
 * ascending order; of rows with equal norms at the threshold the later ones are taken first.  Replaces
 * ZipCacheKVCache._batched_saliency_mask followed by the stable argsort of its mask
 * (veloxquant_mlx/cache/zipcache_cache.py:106-116, 186-190): two stable argsorts and a third over [BH, S]. */
int vq_zip_route(const float *norms, int64_t BH, int64_t S, int64_t n_hi, int32_t *order, void *stream);

/* The round trip along the token axis over ROUTED rows: position s of slab bh stands for row
 * rows[bh * rows_stride + s] of x and of out (both [BH, *, D] with element stride stride_bh between slabs);
 * groups of `group` consecutive positions are quantised together and every reconstructed row is written
 * where its source row lies; rows that no position names are left alone.  Replaces, in one launch and
 * without the gathered copy, the gather -> _group_quant_dequant_batched -> scatter of one salience block
 * of ZipCacheKVCache._compress_tensor (veloxquant_mlx/cache/zipcache_cache.py:118-244): the caller passes
 * the low or the high block's slice of its routing order.  head_dim 64 / 128 / 256. */
int vq_kivi_quant_dequant_rows(const void *x, void *out, int dtype, int64_t BH, int64_t n_rows, int64_t D,
                               int64_t stride_bh, const int32_t *rows, int64_t rows_stride, int group,
                               int levels, float eps, void *stream);

/* Quantise and bit-pack.  Codes follow _quant_keys/_quant_values
 * (benchmark_scripts/benchmark_real_model_scalar_attend.py:115-153;
 * veloxquant_mlx/quantizers/_quant_utils.py:9-46) and the word image follows
 * _pack_indices (veloxquant_mlx/cache/turboquant_rvq_cache.py:82-106).
 *
 * x: [BH, S, D] with row stride D and a per-(b,h) stride of x_stride_bh
 * elements.  Results land at token offset dst_tok0 of destination buffers that
 * hold cap_tokens tokens per (b,h):
 *   axis TOKEN  (keys):   packed [BH, cap_tokens, W], scale/zero
 *                         [BH, ceil(cap_tokens/group), D]; dst_tok0 % group == 0
 *   axis CHANNEL (values), v_layout CHANNEL_PACKED: packed [BH, cap_tokens, W],
 *                         scale/zero [BH, cap_tokens, GV]
 *   axis CHANNEL (values), v_layout TOKEN_PACKED: packed [BH, cap_tokens/per, D],
 *                         scale/zero [BH, GV, cap_tokens]; dst_tok0, S and
 *                         cap_tokens multiples of per
 * W = ceil(D/per), per = 32/pack_bits, GV = ceil(D/group).  pack_bits == 8
 * yields plain uint8 codes.  levels is the top code (2^b - 1 <= 2^pack_bits-1).
 * scale/zero are written as meta_dtype (VQ_F32 exact, VQ_F16 rounded). */
int vq_kivi_quant_pack(const void *x, int dtype, int64_t BH, int64_t S, int64_t D,
                       int64_t x_stride_bh, int axis, int group, int levels, float eps,
                       int pack_bits, int v_layout, void *packed, void *scale, void *zero,
                       int meta_dtype, int64_t cap_tokens, int64_t dst_tok0, void *stream);

/* Keys and values of the same S tokens in one call: vq_kivi_quant_pack of k along the TOKEN
 * axis and of v along the CHANNEL axis in v_layout, into destination buffers of the same
 * cap_tokens at the same dst_tok0 -- the pair of calls every flush of a cache makes
 * (KIVIKVCache.update_and_fetch, veloxquant_mlx/cache/kivi_cache.py:242-262, quantises keys and
 * values of one block back to back).  One launch where D == 128, the inputs are fp16 or bf16
 * and the shapes meet the alignment rules above; otherwise the two single calls. */
int vq_kivi_quant_pack_kv(const void *k, const void *v, int dtype, int64_t BH, int64_t S, int64_t D,
                          int64_t x_stride_bh, int group, int levels, float eps, int pack_bits,
                          int v_layout, void *k_packed, void *k_scale, void *k_zero, void *v_packed,
                          void *v_scale, void *v_zero, int meta_dtype, int64_t cap_tokens,
                          int64_t dst_tok0, void *stream);

/* Packed codes -> reconstruction, out[BH, S, D] = cast(code*scale + zero).
 * Replaces scalar_decode_once(codes, scale, zero, group_size, mode)
 * (veloxquant_mlx/metal/_scalar_attend.py:650-699).  Source buffers are laid
 * out as vq_kivi_quant_pack writes them; tokens [src_tok0, src_tok0+S). */
int vq_kivi_dequant(const void *packed, const void *scale, const void *zero, int meta_dtype,
                    int64_t BH, int64_t S, int64_t D, int axis, int group, int pack_bits,
                    int v_layout, int64_t cap_tokens, int64_t src_tok0, void *out, int out_dtype,
                    void *stream);

/* Appends S new tokens of keys and values, [B, H, S, D] each with element strides
 * k_strides / v_strides = {batch, head, token} and contiguous channels, to the
 * un-quantised tails [B, H, tail_cap, D] (contiguous) at token `pos`, both in one
 * launch.  elem_bytes is 2 (fp16, bf16) or 4; D * elem_bytes and every stride in
 * bytes must be multiples of 16 and every pointer 16-byte aligned.  This is the
 * concatenation step of KIVIKVCache.update_and_fetch
 * (veloxquant_mlx/cache/kivi_cache.py:206-260) into a buffer that already has room. */
int vq_kv_tail_append(const void *k_new, const void *v_new, const int64_t k_strides[3], const int64_t v_strides[3],
                      void *k_tail, void *v_tail, int elem_bytes, int64_t B, int64_t H, int64_t S, int64_t D,
                      int64_t tail_cap, int64_t pos, void *stream);

/* A whole chunk of a packed KIVI cache in one call: the concatenation, the quantisation of
 * the tokens that aged out of the fp16 residual window and the start of the next tail
 * (KIVIKVCache.update_and_fetch, veloxquant_mlx/cache/kivi_cache.py:206-262, on packed
 * buffers).  In stream order:
 * With n_flush == 0 the call is vq_kv_tail_append: k_new / v_new [B, H, S, D] (strides as
 * there) go to rows [n_tail, n_tail + S) of the tails [B, H, tail_cap, D].  With n_flush > 0,
 * of the rows of [tail ; new]
 *   1. the first n_flush are quantised and packed as tokens [dst_tok0, dst_tok0 + n_flush) of
 *      the packed store (keys per channel over token groups, values per token over channel
 *      groups in v_layout; buffers, cap_tokens and the alignment rules are those of
 *      vq_kivi_quant_pack; new rows among them pass through the tails, which must have room
 *      for n_tail + S rows), in one launch for keys and values where D == 128, and
 *   2. the n_tail + S - n_flush rows that stay are written to the front of the spare tails
 *      [B, H, spare_cap, D], which the caller uses as the tails from then on (the old tails'
 *      contents are unspecified afterwards).
 * dtype is the element type of the new tokens and of all four tail buffers. */
typedef struct vq_kivi_append_args {
    const void *k_new, *v_new;
    int64_t k_strides[3], v_strides[3];
    int dtype;
    int64_t B, H, S, D;
    void *k_tail, *v_tail;
    int64_t tail_cap, n_tail;
    int64_t n_flush;
    void *k_packed, *k_scale, *k_zero, *v_packed, *v_scale, *v_zero;
    int meta_dtype;
    int64_t cap_tokens, dst_tok0;
    int group, levels;
    float eps;
    int pack_bits, v_layout;
    void *k_spare, *v_spare;
    int64_t spare_cap;
} vq_kivi_append_args;
int vq_kivi_cache_append(const vq_kivi_append_args *args, void *stream);

/* ---- bit packing ----------------------------------------------------------- */

/* Trailing-axis word packing, idx[rows, D] uint8 <-> words[rows, ceil(D/per)].
 * Replaces _pack_indices/_unpack_indices
 * (veloxquant_mlx/cache/turboquant_rvq_cache.py:82-126). bits in 1..8. */
int vq_pack_words(const uint8_t *idx, int64_t rows, int64_t D, int bits, uint32_t *words, void *stream);
int vq_unpack_words(const uint32_t *words, int64_t rows, int64_t D, int bits, uint8_t *idx, void *stream);

/* Flat byte packing, 8/bits codes per byte, LSB first; bits in {1,2,4}.
 * Replaces turboquant_bit_pack / turboquant_bit_unpack
 * (veloxquant_mlx/metal/_bit_packing.py:87-148). n = number of codes. */
int vq_bit_pack(const uint8_t *idx, int64_t n, int bits, uint8_t *packed, void *stream);
int vq_bit_unpack(const uint8_t *packed, int64_t n, int bits, uint8_t *idx, void *stream);

/* ---- VecInfer product VQ -------------------------------------------------- */

/* Nearest-centroid assignment with one codebook shared by all sub-vectors:
 * x [N, sub_dim] (any float dtype), codebook [n_centroids, sub_dim]; distance
 * sum_i (x_i - c_i)^2 in float32, dimensions added left to right, strict '<'
 * so the lowest index wins ties.  idx_dtype VQ_I32, VQ_U32 or VQ_U8
 * (n_centroids <= 256).  Replaces quantize_vq
 * (veloxquant_mlx/allocators/vecinfer.py:281-318) and vecinfer_quantize_metal
 * (veloxquant_mlx/metal/_vecinfer.py:181-222). */
int vq_vecinfer_assign(const void *x, int x_dtype, int64_t N, const void *codebook, int cb_dtype,
                       int n_centroids, int sub_dim, void *idx, int idx_dtype, void *stream);

/* Fused key encode (+ optional decode) in one launch: keys [B, H, S, D] (any float dtype,
 * contiguous) -> k~ = (keys / smooth) @ Hd with Hd the orthonormal Sylvester-Hadamard matrix
 * of size D (entries +-hadamard_scale, natural order; done as a fast Walsh-Hadamard
 * transform) -> idx [B, H, S, D / sub_dim] by the rule of vq_vecinfer_assign.  smooth is
 * float32 [smooth_rows, D] with smooth_rows 1 or H, or NULL.  k_hat, when not NULL, receives
 * the reconstruction (codebook[idx] @ Hd^T) * smooth in the dtype of keys; k_tilde, when not
 * NULL, receives k~ as float32.  Covers sub_dim 4 or 8, D / sub_dim in {8, 16, 32, 64},
 * n_centroids <= 256, 16-byte aligned buffers; VQ_ERR_UNSUPPORTED otherwise (callers then
 * transform with a matrix product and call vq_vecinfer_assign).  Replaces
 * vecinfer_encode_decode_metal (veloxquant_mlx/metal/_vecinfer.py:225-293,
 * metal/src/vecinfer_encode_decode_full.metal) and the encode half of
 * VecInferKVCache._encode_decode_keys (cache/vecinfer_cache.py:313-356). */
int vq_vecinfer_encode_keys(const void *keys, int k_dtype, int64_t B, int64_t H, int64_t S, int64_t D,
                            const float *smooth, int smooth_rows, float hadamard_scale, const void *codebook,
                            int cb_dtype, int n_centroids, int sub_dim, void *idx, int idx_dtype, void *k_hat,
                            float *k_tilde, void *stream);

/* Centroid gather, out [N, sub_dim] = codebook[min(idx, n_centroids-1)].
 * Replaces dequantize_vq (allocators/vecinfer.py:321-335) and
 * vecinfer_dequant_metal (metal/_vecinfer.py:144-178). */
int vq_vecinfer_dequant(const void *idx, int idx_dtype, int64_t N, const void *codebook,
                        int cb_dtype, int n_centroids, int sub_dim, void *out, int out_dtype,
                        void *stream);

/* ---- attention over a packed KIVI cache ------------------------------------ */

typedef struct vq_attend_args {
    /* queries / output: [B, Hq, Sq, D] contiguous */
    const void *q;
    void *out;
    int q_dtype;   /* VQ_F16 / VQ_BF16 / VQ_F32 */
    int out_dtype; /* VQ_F16 / VQ_BF16 / VQ_F32 */
    int64_t B, Hq, Hkv, Sq, D;
    /* quantised prefix: n_packed tokens laid out as vq_kivi_quant_pack writes
     * them (keys TOKEN axis, values CHANNEL axis in v_layout), buffers sized
     * for cap_tokens tokens per (b, h_kv).  n_packed == 0 is allowed. */
    const void *k_packed, *k_scale, *k_zero;
    const void *v_packed, *v_scale, *v_zero;
    int pack_bits, group, meta_dtype, v_layout;
    int64_t n_packed, cap_tokens;
    /* un-quantised tail: n_tail tokens, [B, Hkv, tail_cap, D], tail_dtype
     * VQ_F16 / VQ_BF16 / VQ_F32.  n_tail == 0 is allowed. */
    const void *k_tail, *v_tail;
    int tail_dtype;
    int64_t n_tail, tail_cap;
    float scale; /* softmax scale applied to q.k */
    int causal;  /* 1: query i sees slots <= n_packed + n_tail - Sq + i */
    int num_splits; /* 0 = choose; > 0 the split count along tokens; < 0 choose, but take the
                     * layout-agnostic vector kernel even where the MFMA kernel applies
                     * (cross-checks of the two implementations); -2: that kernel with every
                     * reconstructed key and value rounded to fp16 first, the form in which the
                     * reference's cache holds them (cache/kivi_cache.py:198-201) and the
                     * 256-row prefill blocks attend over them */
    void *workspace;
    size_t workspace_bytes;
    void *stream;
    /* Optional: int32 counters, one per (sequence, kv head, row tile of the decode path) -- B*Hkv for
     * single-query calls, B*Hkv*ceil(Sq / positions per tile) for multi-query ones, at most B*Hkv*Sq --
     * all zero when the call is enqueued; the call leaves them zero.  With them the MFMA decode path finishes in a single launch (the last
     * block of every kv head merges the split partials); without them (NULL) a separate
     * merge kernel follows.  Calls sharing counters must not overlap. */
    int32_t *sync_counters;
    /* Optional, both or neither: per-sequence lengths for a batch whose sequences differ in
     * length (device arrays of B int32).  Sequence b attends over its first packed_lens[b]
     * packed tokens (a multiple of 32 and of group, <= n_packed) and its first tail_lens[b]
     * tail tokens (<= n_tail); n_packed and n_tail are then the maxima over the batch, which
     * size the launch.  With causal != 0 the queries of sequence b align to the end of its own
     * tokens.  No counterpart in the reference, whose caches carry one offset for the batch
     * (variable-length batches are the integration it scoped and left open,
     * docs/KV_KERNEL_ROOFLINE_FINDINGS.md:963-973). */
    const int32_t *packed_lens;
    const int32_t *tail_lens;
    /* Optional, both or neither: the newest token's key and value rows, [B, Hkv, D] contiguous in
     * tail_dtype, 16-byte aligned.  The call first stores them as the LAST of the n_tail tail rows
     * (row n_tail - 1, or tail_lens[b] - 1) and attends over them from these buffers, so a decode
     * step appends and attends in one launch.  Single-query MFMA decode path only (Sq == 1, what
     * vq_kivi_attend_plan reports as path 1); VQ_ERR_UNSUPPORTED otherwise -- append with
     * vq_kv_tail_append first.  Stands for the concatenation in KIVIKVCache.update_and_fetch
     * (cache/kivi_cache.py:206-260) followed by the attention call of the same step. */
    const void *k_new;
    const void *v_new;
    /* Order in which the decode kernel's waves take token chunks, for this call:
     * 0 = the process default (vq_kivi_attend_fixed_order), 1 = a fixed order (identical bits
     * from run to run), 2 = on demand (fastest; the last bits can differ between runs). */
    int32_t fixed_order;
    /* > 0: a query at position p of the sequence (queries align to the end of the slots) sees
     * only the slots (p - sliding_window, p], with or without `causal` -- the window of
     * VecInferKVCache.fused_sdpa(..., sliding_window) (veloxquant_mlx/cache/vecinfer_cache.py:670-731,
     * metal/src/fused_sdpa.metal).  Whole stretches of packed tokens below the window of every
     * query are not read. */
    int64_t sliding_window;
    /* Protected rows of a sink-protecting cache (SinkProtectedKVCache,
     * veloxquant_mlx/cache/sink_cache.py:117-198, on packed storage -- the reference keeps such rows
     * exact inside its fp16 history and has no packed form).  The packed store holds a stand-in at
     * every protected position (the neighbouring row that took its place when the group was
     * quantised) whose value scale and zero are 0, so it adds nothing to the output sums; the exact
     * rows sit here: sink_k / sink_v [B, Hkv, sink_cap, D] in sink_dtype, sink_pos int32
     * [B, sink_cap] with the position of each row in its sequence (-1: unused slot; positions are
     * below n_packed).  After the attention kernels a patch pass takes the stand-ins' weights out of
     * every query row's softmax sum and puts the exact rows in, under the same causal / window
     * visibility.  NULL sink_k: none. */
    const void *sink_k, *sink_v;
    const int32_t *sink_pos;
    int64_t sink_cap;
    int32_t sink_dtype;
    /* Optional: all n_packed + n_tail slots once more as ready-made fp16 tiles, written by
     * vq_kivi_prefill_tiles: [B * Hkv, tile_cap, VQ_PREFILL_TILE_BYTES], 16-byte aligned, tile u holding
     * slots 32 u .. 32 u + 31 (packed slots reconstructed and rounded to fp16 as the reference's cache
     * holds them, cache/kivi_cache.py:198-201; tail slots as they are).  A multi-query call of 256 or more
     * rows per kv head (prefill chunks) then copies tiles straight into on-chip memory instead of
     * reconstructing the prefix in every block; the results are the same bit for bit.  Other calls ignore
     * it, and so does a call with packed_lens (vq_kivi_attend_plan reports path 2 and 256 or more rows
     * per kv head for the calls that read it).  The cache arrays above must still be given.  No counterpart
     * in the reference (whose memory-bound mode dequantises the whole history to fp16 per call,
     * cache/kivi_cache.py:262-332); a scratch of the prefill phase, 608 bytes per slot and kv head. */
    const void *kv_tiles;
    int64_t tile_cap;
    /* With kv_tiles, for vq_kivi_attend: tiles from this unit on are not up to date; a call that reads the tiles
     * writes them first (as vq_kivi_prefill_tiles would, same stream); a call that does not read them leaves them
     * alone, so a caller learns from vq_kivi_attend_plan (path 2) whether they are up to date afterwards.  A value at or past the number of units: nothing to write. */
    int64_t tiles_stale_from;
} vq_attend_args;

#define VQ_PREFILL_TILE_BYTES 19456

/* Writes tiles first_unit .. first_unit + n_units - 1 of every (sequence, kv head) into a->kv_tiles from the
 * cache arrays of *a (k_packed .. v_zero, n_packed, cap_tokens, k_tail, v_tail, n_tail, tail_cap, B, Hkv, D,
 * stream; the query-side fields are ignored).  D = 128, 2- or 4-bit codes, groups of 32 / 64 / 128, values
 * token-packed, fp16 or bf16 tail, no packed_lens; tiles past ceil((n_packed + n_tail) / 32) are refused.
 * A caller that appends chunk by chunk rewrites only the units that changed: those that were tail slots
 * before the last flush, and the tail.  One launch. */
int vq_kivi_prefill_tiles(const vq_attend_args *a, int64_t first_unit, int64_t n_units);

/* The decode kernel balances its waves by handing out token chunks on demand, so the order in
 * which partial sums are formed, and with it the last bits of the output, can differ from one
 * run to the next (well inside the 2e-3 bar).  enable != 0 changes the process default, which
 * calls with vq_attend_args.fixed_order == 0 take: chunks are dealt in a fixed order instead,
 * identical bits from run to run, a few percent slower.  Returns the previous setting.  No
 * counterpart in the reference (its kernels use a fixed split order); for callers that compare
 * runs bit for bit. */
int vq_kivi_attend_fixed_order(int enable);

/* Bytes of scratch vq_kivi_attend needs for these shapes (fields other than the shapes, pack_bits,
 * group, num_splits, sliding_window and sink_k are ignored).  0 for a launch that writes its output
 * itself (a prefill whose row tiles fill the GPU, one run per row, no protected rows): workspace may
 * then be NULL.  A call with several query positions (fewer than 256 rows a kv head) and a GQA group of 3, 5, 6 or 7 heads runs as
 * the next group size the matrix-unit kernels tile (4 or 8: every group filled up with heads of
 * zeros, whose rows are computed and dropped), a prefill-sized one with more than eight heads a
 * group as passes of eight heads; its queries and outputs in that form are part of
 * this figure, and the workspace must then be 256-byte aligned, q and out 16-byte aligned. */
size_t vq_kivi_attend_workspace(const vq_attend_args *a);

/* Reports what vq_kivi_attend would do for these arguments: *path = 0 for the
 * layout-agnostic vector kernel, 1 for the MFMA decode kernel, 2 for the MFMA
 * prefill kernel (16 or more queries per sequence); *nparts = number of partial
 * results per query row.  No counterpart in the reference (its
 * _auto_nsg heuristic, veloxquant_mlx/metal/_scalar_attend.py:337-362, is the
 * nearest thing); used by tests and benchmarks to name the kernel measured. */
int vq_kivi_attend_plan(const vq_attend_args *a, int *path, int *nparts);

/* softmax(q k^T * scale) v over [quantised prefix | tail] with GQA by
 * repeat-interleave (query heads [h*Hq/Hkv, (h+1)*Hq/Hkv) share kv head h).
 * Sq == 1, causal == 0 replaces scalar_fused_decode_attend
 * (veloxquant_mlx/metal/_scalar_attend.py:370-493); a leading layer axis of
 * scalar_fused_decode_attend_batched (:496-647) folds into B; n_packed == 0
 * replaces scalar_predecoded_attend (:702-779) and, with causal == 1,
 * flash_prefill_attend (veloxquant_mlx/metal/_flash_prefill.py:171-237). */
int vq_kivi_attend(const vq_attend_args *a);

/* vq_kivi_attend for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * split partials and the sync counters come from a device array built into the library (8 MiB +
 * 64 KiB per GPU, held until the process ends); a->workspace, a->workspace_bytes and
 * a->sync_counters are ignored.  Shapes whose partials exceed 8 MiB (vq_kivi_attend_workspace) or
 * with more than 16384 (sequence, kv head, row tile) triples return VQ_ERR_WORKSPACE.  The call
 * itself allocates and frees nothing.  All calls on one GPU share that GPU's array: calls that
 * overlap on one GPU (two streams, two threads) race -- serialise them, or use vq_kivi_attend
 * with a workspace per stream.  The first call on a device looks the array's address up, and the
 * first launch of each kernel instantiation raises its block-shared-memory limit: make one call
 * per device and shape class (bit width, group size, scale type, rows per kv head) outside any
 * stream capture before capturing.  A call that fails clears the shared counters behind itself. */
int vq_kivi_attend_static(const vq_attend_args *a);

/* ---- attention over VecInfer indices ----------------------------------------- */

typedef struct vq_lut_attend_args {
    /* transformed queries (apply_dual_transform_queries already applied) / output:
     * [B, Hq, Sq, D] contiguous */
    const void *q;
    void *out;
    int32_t q_dtype, out_dtype;
    int64_t B, Hq, Hkv, Sq, D;
    /* codebook indices [B, Hkv, cap_tokens, D / sub_dim], VQ_U8, VQ_I32 or VQ_U32; the first
     * n_tokens tokens are live */
    const void *k_idx, *v_idx;
    int32_t idx_dtype;
    int64_t n_tokens, cap_tokens;
    /* codebooks [n_centroids, sub_dim] shared by every sub-vector position */
    const void *k_codebook, *v_codebook;
    int32_t cb_dtype;
    int32_t n_centroids, k_sub_dim, v_sub_dim;
    float scale;
    int32_t causal;          /* queries align to the end of the tokens */
    int64_t sliding_window;  /* > 0: a query sees only that many last tokens before its position */
    int32_t num_splits;      /* 0 = choose */
    void *workspace;         /* at least vq_vecinfer_attend_workspace(args) bytes */
    size_t workspace_bytes;
    void *stream;
} vq_lut_attend_args;

/* softmax((q~ k~^T) * scale) v^ computed from the indices with a per-query look-up table
 * (scores) and a per-query histogram over centroids (values); neither k~^ nor v^ is
 * materialised.  Covers n_centroids <= 256, D / sub_dim <= 32 and
 * (D / k_sub_dim + D / v_sub_dim) * n_centroids * 4 <= 64 KB; other shapes return
 * VQ_ERR_UNSUPPORTED.  Replaces metal_fused_sdpa
 * (veloxquant_mlx/metal/fused_sdpa.py:200-299, fused_sdpa.metal) under
 * VecInferKVCache.fused_sdpa (veloxquant_mlx/cache/vecinfer_cache.py:670-731). */
size_t vq_vecinfer_attend_workspace(const vq_lut_attend_args *a);
int vq_vecinfer_attend(const vq_lut_attend_args *a);

/* ---- SKVQ clipped group quantisation ------------------------------------- */

/* Round trip of rows through per-token, per-channel-group asymmetric quantisation with a
 * grid-searched clip factor: out = cast(code*scale + lo) under the first of `alphas` with the
 * smallest group error.  Replaces clipped_group_quant followed by clipped_group_dequant
 * (veloxquant_mlx/quantizers/skvq.py:105-183) together with the channel gather and inverse
 * gather around them in SKVQKVCache._round_trip (veloxquant_mlx/cache/skvq_cache.py:236-251).
 * x/out: B*H slabs of [r, D] rows, slab b*H+h at element offset (b*H+h)*stride_bh; same dtype;
 * out may alias x.  perm: device int32 [H, D] channel order per head, or NULL for the identity.
 * inv: optional device int32 [H, D] inverse of perm (inv[h][perm[h][j]] = j); with it rows move as
 * 16-byte pieces under a channel order too (results are the same).
 * alphas: host array of n_alphas (1..8) clip factors in (0, 1]. */
int vq_skvq_clipped_roundtrip(const void *x, void *out, int dtype, int64_t B, int64_t H, int64_t r, int64_t D,
                              int64_t x_stride_bh, int64_t out_stride_bh, const int32_t *perm, const int32_t *inv,
                              int bits, int group, const float *alphas, int n_alphas, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* VELOXQUANT_HIP_H */
