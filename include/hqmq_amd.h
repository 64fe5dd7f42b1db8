/* hqmq_amd.h — C ABI of libhqmq_amd.so: the HQMQ KV-cache path on MI355X (gfx950).
 *
 * Every entry point takes raw device pointers, explicit sizes and a HIP stream
 * (void*, NULL = the null stream), enqueues its kernels on that stream and
 * returns without synchronising.  The library allocates nothing: outputs and
 * scratch are caller-owned device buffers.  Return value: 0 = ok, negative =
 * argument error (hqmq_status_string explains), positive = hipError_t.
 *
 * The reference is pure Python (PyTorch + Triton) and has no FFI; each entry
 * point names the reference function whose work it replaces.  A Python caller
 * binds these with ctypes (see hqmq_amd/_lib.py).
 *
 * Element types: HQMQ_F32 / HQMQ_F16 / HQMQ_BF16 name the dtype D of the K/V
 * tensor.  All arithmetic that decides an integer (codeword index, radius
 * code, Med3x mask) reproduces torch's CPU rounding in D.
 *
 * Packed cache layout (one "plane set" per tensor K or V of one layer), all
 * planes contiguous [B][H][t_cap][row]:
 *   code      = idx | rq << idx_bits,  idx_bits = ceil(log2(24*S)), rq < 2^radius_bits
 *   main row  = little-endian bit stream of the low main_bits of each of the n codes
 *   aux row   = bit stream of the remaining aux_bits (absent when aux_bits == 0)
 *   scale     = per-token r_max in D
 *   flags row = 1 bit per chunk (Med3x outlier), n/8 bytes            (optional)
 *   sideband  = [B][H][sb_cap][4] in D: the flagged chunks verbatim, in
 *               (token, chunk) order; sb_tile_off[B][H][t_cap/16] = number of
 *               flagged chunks before token 16*i (INT32_MAX for tiles not yet written);
 *               sb_count[B][H] = total; sb_coord[B][H][sb_cap] = (token & 15) << 8 | chunk per entry.
 *               A flagged chunk's code keeps its idx but carries rq = 0, so that
 *               it decodes to exactly zero and only the sideband value counts.
 *   s24_r3 -> 12+1 bits (48+4 B/token at d_h=128), s96_r4 -> 16+0 (64 B),
 *   s192_r6 -> 16+3 (64+12 B).
 */
#ifndef HQMQ_AMD_H
#define HQMQ_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { HQMQ_F32 = 0, HQMQ_F16 = 1, HQMQ_BF16 = 2 };

enum {
    HQMQ_OK = 0,
    HQMQ_ERR_NULL = -1,      /* a required pointer is NULL */
    HQMQ_ERR_SHAPE = -2,     /* a size is out of the supported range */
    HQMQ_ERR_DTYPE = -3,     /* unknown or unsupported dtype */
    HQMQ_ERR_LAYOUT = -4,    /* bit widths inconsistent with the layout rules */
    HQMQ_ERR_WORKSPACE = -5, /* workspace too small */
    HQMQ_ERR_ALIGN = -6,     /* a pointer or stride is not aligned as required */
    HQMQ_ERR_SCRATCH = -7    /* hqmq_attn_fwd_static: the call needs more than the library's static scratch
                                (HQMQ_ATTN_STATIC_SCRATCH_BYTES), or asks for skip_combine */
};

int hqmq_version(void);                    /* 0xMMmmpp */
const char *hqmq_status_string(int status);

/* Bit widths of the packed layout for a codebook of 24*S codewords and
 * radius_bits radius bits.  Any output pointer may be NULL. */
int hqmq_layout_bits(int secondary_size, int radius_bits, int *idx_bits, int *main_bits, int *aux_bits);

/* Joint codebook q_p*q_s in D with the reference's op-by-op rounding, k = p*S + s.
 * Replaces HQMQQuantizer._get_codebook (src/quantizers/hqmq.py:119-143).
 *   raw    [H][S][4] fp32, unnormalised secondary parameters of one (layer, K|V)
 *   joint  [H][24*S][4] in D (out)
 *   slack  [H] fp32 (out): max_k || joint[k] - exact(q_p*q_s) ||_2, the bound the
 *          quantize kernel's candidate filter needs */
int hqmq_build_joint(const float *raw, int H, int S, int dtype, void *joint, float *slack, void *stream);

/* Quantize (and optionally pack) x[B][H][T][4n].
 * Replaces HQMQQuantizer._qdq (src/quantizers/hqmq.py:145-216, unit magnitude,
 * linear radius) and, when thr != NULL, the mask/merge half of
 * OutlierAwareHQMQQuantizer._qdq (src/quantizers/outlier_aware.py:72,86).
 * Any output may be NULL. */
typedef struct hqmq_quantize_args {
    const void *x;            /* D, last dim contiguous */
    int64_t x_stride_b, x_stride_h, x_stride_t; /* in elements */
    int dtype;
    int B, H, T, n_chunks;
    const void *joint;        /* [H][24*S][4] D */
    const float *slack;       /* [H] from hqmq_build_joint */
    int secondary_size, radius_bits;
    int algo;                 /* 0 = closed-form filter + exact re-score, 1 = brute force */
    /* unpacked outputs, contiguous [B][H][T][n] / [B][H][T] / [B][H][T][4n] */
    int32_t *idx_out, *rq_out;
    void *rmax_out;           /* D */
    void *dense_out;          /* D: the reference's fake-quant tensor (outlier chunks restored if thr) */
    /* Med3x: per-head threshold in D; mask = ||chunk|| > thr */
    const void *thr;          /* [H] D or NULL */
    uint8_t *mask_out;        /* [B][H][T][n] bytes or NULL */
    /* packed outputs: row (pos ? pos[b] : 0) + t_off + t of each [B][H][t_cap] plane */
    uint8_t *main_plane, *aux_plane, *flag_plane;
    void *scale_plane;        /* D */
    int64_t t_cap;
    int t_off;
    const int32_t *pos;       /* [B] or NULL */
    int main_bits, aux_bits;
    int32_t *stats;           /* [2] or NULL, accumulated: lanes that scored all rows; secondaries kept by the filter */
    uint32_t *scale_max_bits; /* [1] or NULL, accumulated (atomic max): the largest finite per-token scale written to
                                 scale_plane, as the bits of an fp32 number; start it at 0.  The attention kernels read
                                 it (hqmq_packed.scale_max_bits) to keep caches whose scales lie outside [2^-8, 2^15)
                                 inside the normal fp16 range of their matrix products. */
} hqmq_quantize_args;
int hqmq_quantize(const hqmq_quantize_args *a, void *stream);

/* Med3x statistics: per-head median of the chunk norms of one call and the
 * threshold RNE_D(median * mult).  Replaces the torch.quantile half of
 * OutlierAwareHQMQQuantizer._qdq (src/quantizers/outlier_aware.py:60-69).
 *   workspace  hqmq_med3x_workspace_bytes(H, dtype) bytes, any content
 *   median     [H] fp32 (out);  thr [H] D (out);  n_out [H] int32 (out, may be NULL):
 *              number of chunks with norm > thr */
int64_t hqmq_med3x_workspace_bytes(int H, int dtype);
int hqmq_med3x_threshold(const void *x, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_t, int dtype,
                         int B, int H, int T, int n_chunks, float mult, void *workspace, int64_t workspace_bytes,
                         float *median, void *thr, int32_t *n_out, void *stream);

/* Med3x mask alone, for wrappers around quantizers other than HQMQ: mask[b][h][t][c] = ||chunk|| > thr[h]
 * (src/quantizers/outlier_generic.py:60 of the reference). One byte per chunk. */
int hqmq_outlier_mask(const void *x, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_t, int dtype,
                      int B, int H, int T, int n_chunks, const void *thr, uint8_t *mask, void *stream);

/* Compact the flagged chunks of rows [row0, row0+T) into the sideband.
 * No counterpart in the reference (its wrapper keeps a dense tensor).
 * Rows must be appended in order and each row once; row0 = (pos ? pos[b] : 0) + t_off.  (A row that is
 * compacted a second time leaves its first entries in the list: the attention kernels that walk the list would
 * count them twice.  To rewrite rows, reset sb_count and the tile offsets to the state before them.)
 * sb_coord [B][H][sb_cap] (may be NULL): (row & 15) << 8 | chunk of every sideband entry, which lets the
 * specialised attention kernels walk the sideband densely; sb_tile_off must start out as INT32_MAX (tiles not
 * yet written read as "no entries").
 * A full sideband: *overflow is set to 1, and with `planes` (the packed planes that hqmq_quantize wrote for the
 * same rows) every flagged chunk that finds no room is turned back into a plain chunk: its flag bit is cleared and
 * the radius code the quantizer gives an unflagged chunk is written into its radius field, so that it decodes as
 * plain HQMQ instead of zero (the reference never loses an outlier, src/quantizers/outlier_aware.py:86; here a full
 * sideband costs accuracy, never the chunk).  Without `planes` (NULL) such chunks keep radius code 0 and decode to
 * zero: check *overflow.  hqmq_append_kv always passes the planes. */
typedef struct hqmq_packed_rows {
    uint8_t *main_plane, *aux_plane;  /* as passed to hqmq_quantize (aux_plane NULL when aux_bits = 0) */
    const void *scale_plane;          /* D, [B][H][t_cap] */
    int idx_bits, main_bits, aux_bits, qmax;
} hqmq_packed_rows;
int hqmq_outlier_compact(const void *x, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_t, int dtype,
                         int B, int H, int T, int n_chunks, uint8_t *flag_plane, int64_t t_cap, int t_off,
                         const int32_t *pos, void *sideband, int64_t sb_cap, int32_t *sb_tile_off, int32_t *sb_count,
                         int32_t *overflow, uint16_t *sb_coord, const hqmq_packed_rows *planes, void *stream);

/* One append of new K and V rows to a packed cache: Med3x threshold (when median_mult > 0), quantize + pack,
 * sideband compaction, for both tensors.  The results are those of hqmq_med3x_threshold, hqmq_quantize and
 * hqmq_outlier_compact called in that order for K and then for V (what KVQuantizer.quantize_K / quantize_V of
 * src/quantizers/base.py:19-27 do one after the other, src/model_utils.py:22-32); when K and V have the same shape
 * every stage is one launch shared by the two tensors, and for appends of at most 256 / n_chunks rows (n_chunks a
 * power of two) the quantize launch also does the compaction: a single-token append is two launches, not six.
 *   q            as for hqmq_quantize; with median_mult > 0, q.thr is ignored (thr below is used) and q.flag_plane
 *                is required
 *   median_mult  0: no outlier extraction (the fields below are not read) */
typedef struct hqmq_append_args {
    hqmq_quantize_args q;
    float median_mult;
    void *med_workspace; int64_t med_workspace_bytes;  /* hqmq_med3x_workspace_bytes(H, dtype) */
    float *median; void *thr; int32_t *n_out;          /* [H] outputs: fp32, D, int32 (n_out may be NULL) */
    void *sideband; int64_t sb_cap;
    int32_t *sb_tile_off, *sb_count, *overflow;
    uint16_t *sb_coord;                                /* may be NULL */
} hqmq_append_args;
int hqmq_append_kv(const hqmq_append_args *k, const hqmq_append_args *v, void *stream);

/* Dense decode of unpacked codes: out = joint[h, idx] * ((rq * rs) / qmax) in D.
 * Replaces hqmq_decode_triton (src/quantizers/hqmq_kernel.py:102-132) with the
 * rounding of _decode_kv_torch (src/quantizers/hqmq_attention.py:39-65).
 * Strides in elements; idx/rq last dim contiguous; out contiguous [B][H][T][4n]. */
int hqmq_dequant(const int32_t *idx, int64_t idx_sb, int64_t idx_sh, int64_t idx_st,
                 const int32_t *rq, int64_t rq_sb, int64_t rq_sh, int64_t rq_st,
                 const void *rs, int64_t rs_sb, int64_t rs_sh, int64_t rs_st,
                 const void *joint, int64_t joint_sh, int K, int dtype, int B, int H, int T, int n_chunks,
                 int qmax, void *out, void *stream);

/* Pack unpacked codes into main/aux/scale rows (for callers that hold the
 * reference's int32 representation).  No counterpart in the reference. */
int hqmq_pack_codes(const int32_t *idx, int64_t idx_sb, int64_t idx_sh, int64_t idx_st,
                    const int32_t *rq, int64_t rq_sb, int64_t rq_sh, int64_t rq_st,
                    int B, int H, int T, int n_chunks, int idx_bits, int main_bits, int aux_bits,
                    uint8_t *main_plane, uint8_t *aux_plane, int64_t t_cap, void *stream);

/* One packed tensor (K or V) as the attention and dense-decode kernels read it. */
typedef struct hqmq_packed {
    const uint8_t *main_plane, *aux_plane, *flag_plane; /* aux/flag may be NULL */
    const void *scale_plane;  /* D, or any float dtype given by scale_dtype */
    int64_t scale_sb, scale_sh, scale_st; /* element strides of scale_plane (contiguous: H*t_cap, t_cap, 1) */
    const void *sideband;     /* NULL when flag_plane is NULL */
    const int32_t *sb_tile_off;
    int64_t sb_cap;
    const uint16_t *sb_coord; /* [B][H][sb_cap] entry coordinates, or NULL (then the layout-generic kernel is used) */
    const int32_t *sb_count;  /* [B][H] entries in use */
    const void *joint;        /* [H][K][4] D */
    int64_t joint_sh;         /* element stride between heads */
    int K;                    /* codewords in joint */
    const uint32_t *scale_max_bits; /* [1] or NULL: an upper bound of the finite scales in scale_plane as fp32 bits, as
                                 hqmq_quantize accumulates it.  Read by the layout-generic attention kernel (see
                                 hqmq_attn_args.wide_range): with a bound of 2^15 or more, or below 2^-8, the softmax
                                 weights are carried with a power-of-two offset and verbatim outlier chunks are rescaled,
                                 so that every product stays finite and normal in fp16 (the result is unchanged: numerator
                                 and denominator carry the same factor).  NULL = no offset. */
} hqmq_packed;

/* Dense decode of a packed cache (outlier chunks substituted from the sideband).
 * mode 0: cw * ((rq * rs) / qmax), the rounding of _decode_kv_torch
 *         (src/quantizers/hqmq_attention.py:61-64) that the attention path is checked against;
 * mode 1: (rq * (rs / qmax)) * cw, the rounding of the quantizer's own output
 *         (src/quantizers/hqmq.py:210-216). */
int hqmq_dequant_packed(const hqmq_packed *p, int dtype, int B, int H, int T, int n_chunks, int64_t t_cap,
                        int idx_bits, int main_bits, int aux_bits, int qmax, int mode, void *out, void *stream);

/* Fused attention over the packed cache: decode (T_q = 1) and chunked prefill.
 * Replaces fused_hqmq_attention_triton (src/quantizers/hqmq_attention.py:425-518)
 * with the semantics of fused_hqmq_attention_torch (:68-101).
 * Query row i of sequence b sees key j iff j < kv_len[b] (T_kv when kv_len is
 * NULL) and (not causal or j <= i + causal_offset); causal_offset = 0 is the
 * reference's top-left alignment.
 *   workspace   hqmq_attn_workspace_bytes(...) bytes of scratch for split-KV partials, 16-byte aligned, any content */
typedef struct hqmq_attn_args {
    const void *Q; void *O;   /* D, [B][H_q][T_q][d_h]; strides in elements, last dim contiguous */
    int64_t q_sb, q_sh, q_st, o_sb, o_sh, o_st;
    hqmq_packed K, V;
    int dtype;
    int B, H_q, H_kv, T_q, T_kv, n_chunks;
    int64_t t_cap;
    int idx_bits, main_bits, aux_bits, qmax;
    const int32_t *kv_len;    /* [B] or NULL */
    int causal; int64_t causal_offset;
    float softmax_scale;
    int n_splits;             /* 0 = choose */
    void *workspace; int64_t workspace_bytes;
    int skip_combine;         /* 1: leave the split partials in the workspace (merge later with hqmq_attn_combine) */
    int force_generic;        /* 1: use the layout-generic kernel even where a specialised one exists (testing);
                                 2: keep the specialised kernels that hold their tiles in registers where the kernel that
                                 lands its loads in LDS would run (plain 16+0 caches at d_h 128; identical results) */
    const int32_t *kv_start;  /* [B] or NULL: first visible token of every sequence (left-padded batches) */
    const int32_t *batch_order; /* [B] or NULL: a permutation of 0..B-1, the order in which the sequences' blocks are
                                   started (pass the sequences sorted by length, longest first, for ragged batches) */
    void *start_event, *stop_event; /* hipEvent_t or NULL: receive the GPU timestamps of the begin and the end of
                                       the main attention kernel (hipEventElapsedTime = its duration; profiling) */
    int fp8_table_storage;    /* 1: every entry of both joint tables is a float8 e4m3 number (the caller rounded them, as
                                 the reference's use_fp8_codebook does, src/quantizers/hqmq_attention_hopper.py:43-53) and
                                 the kernel may keep them as float8 in LDS (4 bytes per codeword, widened after the
                                 gather as :133-135 there does).  Same results as 0 on such tables; honoured by the
                                 specialised decode kernels of the 16-bit layouts at d_h 128, ignored elsewhere. */
    int wide_range;           /* 1: a bf16 cache whose per-token scales may reach 2^15 (or whose verbatim outlier values may
                                 exceed 65504), or whose largest scale is below 2^-8.  The specialised kernels multiply the
                                 softmax weights with the V scales in fp16 and would overflow, or lose the product to fp16
                                 subnormals; such a cache takes the layout-generic kernel, which reads
                                 hqmq_packed.scale_max_bits and keeps every product inside the normal fp16 range (fp32 caches
                                 always take it).  Callers that track the bound (hqmq_quantize_args.scale_max_bits) set this
                                 when it leaves [2^-8, 2^15); data of ordinary magnitude never does. */
} hqmq_attn_args;
int64_t hqmq_attn_workspace_bytes(int B, int H_q, int T_q, int d_h, int n_splits);
/* The n_splits hqmq_attn_fwd would choose; ragged = 1 when kv_len is passed (more, smaller blocks). */
int hqmq_attn_pick_splits(int B, int H_q, int H_kv, int T_q, int T_kv, int ragged);
int hqmq_attn_fwd(const hqmq_attn_args *a, void *stream);
/* Merge of the split-KV partials (m, l, acc) left in the workspace; hqmq_attn_fwd runs it unless skip_combine. */
int hqmq_attn_combine(const void *workspace, void *O, int dtype, int B, int H_q, int T_q, int d_h, int n_splits,
                      int64_t o_sb, int64_t o_sh, int64_t o_st, void *stream);

/* hqmq_attn_fwd for callers that cannot allocate or hand over scratch memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments, kernels and results as hqmq_attn_fwd, except that a->workspace / a->workspace_bytes are ignored:
 * the split-KV partials live in a device array of HQMQ_ATTN_STATIC_SCRATCH_BYTES that is part of the library's
 * code object (every GPU the library runs on holds its own copy until the process ends).  The call allocates and
 * frees nothing.  It returns HQMQ_ERR_SCRATCH when hqmq_attn_workspace_bytes(B, H_q, T_q, d_h, n_splits) for the
 * chosen n_splits exceeds that size (every decode shape of the benchmark configurations fits; long chunked
 * prefills do not: pass a smaller n_splits or use hqmq_attn_fwd) and when skip_combine is set.
 * All calls on one GPU share the array: calls that overlap on one GPU (different streams or threads) race.
 * The first call on a device looks the array's address up (hipGetSymbolAddress) and must not be made under
 * stream capture; later calls may be. */
#define HQMQ_ATTN_STATIC_SCRATCH_BYTES (8 << 20)
int64_t hqmq_attn_static_scratch_bytes(void);
int hqmq_attn_fwd_static(const hqmq_attn_args *a, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HQMQ_AMD_H */
