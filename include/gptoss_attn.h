/*
 * gptoss_attn.h -- C ABI of the MI355X (gfx950) GPT-OSS flash-attention library.
 *
 * The reference project has no native layer: its device code is three Triton
 * kernels launched from a torch.autograd.Function (attention_kernel.py:220-344).
 * Each entry point below names the reference code it stands in for, so a
 * maintainer can bind it (ctypes, cffi, a torch custom op) at the same place.
 *
 * Conventions
 *   - plain pointers and sizes only; no torch, no HIP types (the stream is passed
 *     as a void* holding a hipStream_t; NULL is the default stream);
 *   - every buffer is owned by the caller; the library allocates nothing.  Its only
 *     process-wide state is per-device values that are looked up once and never change
 *     (compute-unit count, a kernel attribute, the address of the built-in scratch of
 *     gptoss_attn_bwd_static), so calls on different streams are independent;
 *   - launches are asynchronous on `stream`; no entry point synchronises;
 *   - outputs need no pre-zeroing (the reference needs dk/dv/dsinks zeroed,
 *     attention_kernel.py:296-298; this library writes every element once);
 *   - return value: 0 ok; negative = argument error (table below), checked on
 *     the host before anything is launched; positive = the hipError_t of a
 *     failed launch.  No C++ exception crosses the boundary.
 *
 * Tensors (element strides, innermost head_dim stride fixed at 1):
 *   q, dq        (B, H, Sq, D)     query heads
 *   k, v, dk, dv (B, G, Skv, D)    KV heads; query head h reads KV head h/(H/G)
 *                                  (attention_kernel.py:36,152)
 *   o, d_o       (B, Sq, H, D) by default in the caller's view, but addressed
 *                through the same (b, h, s) stride triple, so any layout works
 *   lse          (B, H, Sq) fp32 contiguous
 *   delta        fp32 scratch of gptoss_attn_workspace_bytes() bytes, 16-byte aligned: -rowsum(dO*O), then
 *                lse*log2(e), then both once more as 16 bytes per row of bf16 terms for the dK/dV
 *                kernels, then (short sequences) partial dK/dV sums
 *   sinks, dsinks (H,) fp32;  sinks == NULL means a sink logit of 0, as in the
 *                reference (attention_kernel.py:39-42)
 *   seqlens      (B,) int32 or NULL: right-padding lengths.  Keys at or beyond
 *                seqlens[b] are invisible; query rows at or beyond it produce
 *                O = 0, lse = sink and contribute no gradient.
 *   doc_start    (B, Sq) int32 or NULL, for rows packed from several documents:
 *                doc_start[b][i] is the index of the first token of the document
 *                that query i belongs to (non-decreasing along i); keys before it
 *                are invisible.  Needs Sq == Skv and q_offset == 0.  NULL (what
 *                the reference does, it ignores position ids) lets documents of a
 *                packed row see each other.
 * Visibility of key j to the query at absolute position p = q_offset + i:
 *   j <= p  and  (window == 0 or j > p - window)      (attention_kernel.py:68,71)
 */
#ifndef GPTOSS_ATTN_H
#define GPTOSS_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GPTOSS_ATTN_ABI_VERSION 4

enum gptoss_attn_dtype {
    GPTOSS_ATTN_BF16 = 0, /* 2-byte bfloat16 tensors, bf16 MFMA products, fp32 accumulation: the fast path */
    GPTOSS_ATTN_FP32 = 1  /* 4-byte float tensors, fp32 MFMA products (the reference's fp32 mode,
                             attention_kernel.py is dtype-generic): built for exactness, not tuned */
};

enum gptoss_attn_status {
    GPTOSS_ATTN_OK = 0,
    GPTOSS_ATTN_ERR_NULL_PARAMS = -1,   /* params pointer is NULL */
    GPTOSS_ATTN_ERR_NULL_TENSOR = -2,   /* a required tensor pointer is NULL */
    GPTOSS_ATTN_ERR_HEAD_DIM = -3,      /* D != 64 */
    GPTOSS_ATTN_ERR_HEADS = -4,         /* H <= 0, G <= 0 or H % G != 0 */
    GPTOSS_ATTN_ERR_SHAPE = -5,         /* B, Sq or Skv <= 0, window < 0, q_offset < 0, scale <= 0,
                                           Sq + q_offset, Skv or window above 2^30, doc_start with
                                           Sq != Skv or q_offset != 0, or a launch of more than
                                           2^31-1 workgroups */
    GPTOSS_ATTN_ERR_DTYPE = -6,         /* dtype not in gptoss_attn_dtype */
    GPTOSS_ATTN_ERR_ALIGNMENT = -7,     /* a tensor base or stride breaks 16-byte row alignment */
    GPTOSS_ATTN_ERR_STRIDE = -8,        /* a sequence stride smaller than D or larger than 2^24 elements */
    GPTOSS_ATTN_ERR_ABI = -9,           /* struct_size does not match this library */
    GPTOSS_ATTN_ERR_WORKSPACE = -10     /* gptoss_attn_bwd_static: 24*B*H*Sq bytes do not fit the built-in scratch */
};

/* Size of the device array gptoss_attn_bwd_static keeps its row statistics in: 24 bytes per row must
 * fit, i.e. B*H*Sq <= 2 097 152 rows (the 64-head layer at S = 16384 is 1 048 576 rows per batch row). */
#define GPTOSS_ATTN_STATIC_SCRATCH_BYTES (48u << 20)

/* (batch, head, sequence) strides in elements. */
typedef struct gptoss_attn_strides {
    int64_t b, h, s;
} gptoss_attn_strides;

typedef struct gptoss_attn_params {
    uint32_t struct_size;   /* sizeof(gptoss_attn_params), checked by every call */
    int32_t dtype;          /* gptoss_attn_dtype of q,k,v,o,d_o,dq,dk,dv */

    int32_t B, H, G, Sq, Skv, D;
    int32_t window;         /* 0 = full causal; else sliding window length */
    int32_t q_offset;       /* absolute position of query row 0 (reference start_q) */
    float scale;            /* softmax scale (reference sm_scale) */
    int32_t reserved0;

    const void *q, *k, *v;
    const float *sinks;     /* optional */
    const int32_t *seqlens; /* optional */
    const int32_t *doc_start; /* optional */
    void *o;
    float *lse;

    const void *d_o;
    void *dq, *dk, *dv;
    float *dsinks;          /* optional: NULL skips the sink gradient */
    float *delta;           /* fp32 scratch of gptoss_attn_workspace_bytes() bytes */

    gptoss_attn_strides q_stride, k_stride, v_stride, o_stride;
    gptoss_attn_strides do_stride, dq_stride, dk_stride, dv_stride;

    /* Optional: device address of one int32 holding the absolute position of query row 0.  When set,
     * q_offset above is ignored and the kernels read the value themselves (one scalar load per
     * workgroup), so a caller whose start position lives on the device (the reference reads its
     * `start_q` tensor inside the kernels, attention_kernel.py:44-47,145-147) neither synchronises
     * nor bakes the value into a captured graph.  The value must satisfy 0 <= value and
     * Sq + value <= 2^30 (the kernels clamp it into that range); the host cannot see it, so a window
     * that covers the whole row is not recognised as full causal, the single-pass window backward
     * is not taken, and doc_start is refused (ERR_SHAPE). */
    const int32_t *q_offset_dev;
} gptoss_attn_params;

/* Library/ABI version (GPTOSS_ATTN_ABI_VERSION it was built with). */
int gptoss_attn_version(void);

/* Text for a status code returned by any entry point (never NULL). */
const char *gptoss_attn_status_string(int status);

/*
 * Bytes of the `delta` scratch buffer the backward entry points need for these shapes; 0 for a
 * NULL or shapeless params.  Reads dtype, B, H, G, Sq, Skv and window.  The buffer holds
 * 24 bytes of row statistics per (batch, head, query row): 2 * B * H * Sq floats, and the same numbers
 * (lse / scale and -delta) each split into three bf16 terms, which the dK/dV kernels feed to the matrix
 * pipe as one more step of their S and dP products.  When the problem has too few key blocks to fill the
 * GPU (bf16, full-causal, short sequences), the fp32 partial dK / dV sums of the slices each key
 * block is cut into.  The reference allocates its counterpart itself
 * (`delta = torch.empty_like(M)`, attention_kernel.py:303) and accumulates dK / dV with atomics
 * (:204,212); here the caller owns the scratch and the sums are taken in a fixed order.  For the
 * sliding-window layers that gptoss_attn_bwd runs as one kernel the same bytes hold that kernel's
 * dSinks partial sums and the fp32 dK / dV shares of the key tiles on the seams between workgroups;
 * how many seams there are depends on the compute-unit count of the device the launch runs on, and
 * the size returned covers the largest number any device can ask for.  Host-only: no HIP call.
 */
size_t gptoss_attn_workspace_bytes(const gptoss_attn_params *params);

/*
 * Forward: O and logsumexp.  Replaces the `_attn_fwd` launch in
 * `_attention.forward` (attention_kernel.py:11-100, 241-262) including the
 * output transpose copy at :272 (O is written directly in the caller's layout).
 * Reads q,k,v,sinks,seqlens,doc_start; writes o,lse.
 */
int gptoss_attn_fwd(const gptoss_attn_params *params, void *stream);

/*
 * Backward step 1: the row statistics.  The first B*H*Sq floats of `delta` receive
 * -rowsum(dO * O) (the NEGATED row dot: it seeds the dP accumulators of the kernels that
 * follow), the next B*H*Sq floats lse * log2(e); behind them (from the next 16-byte boundary) 16
 * bytes per row hold lse / scale and the negated row dot as three bf16 terms each, the form the dK/dV
 * kernels read.  Replaces `_attn_bwd_precompute_D`
 * (attention_kernel.py:102-120, 304-313) including the dO transpose copy at
 * :290.  When dsinks != NULL it also produces
 * dsinks[h] = -sum_{b,i} exp(sinks[h] - lse) * delta   (attention_kernel.py:173-176)
 * without atomics.  Reads o,d_o,lse,sinks; writes delta,dsinks.
 */
int gptoss_attn_bwd_preprocess(const gptoss_attn_params *params, void *stream);

/*
 * Backward step 2: dK and dV, KV-outer, no atomics (deterministic).  Replaces
 * the dv/dk halves of `_attn_bwd` (attention_kernel.py:199-212).
 * Reads q,k,v,d_o,lse,delta,seqlens,doc_start; writes dk,dv.
 */
int gptoss_attn_bwd_dkdv(const gptoss_attn_params *params, void *stream);

/*
 * Backward step 3: dQ.  Replaces the dq half of `_attn_bwd`
 * (attention_kernel.py:206-217).  Reads q,k,v,d_o,lse,delta,seqlens,doc_start; writes dq.
 */
int gptoss_attn_bwd_dq(const gptoss_attn_params *params, void *stream);

/*
 * Whole backward on one stream, i.e. `_attention.backward`
 * (attention_kernel.py:276-344).  bf16 tensors take one of two routes:
 *   - sliding-window layers with window <= 128, Sq == Skv, q_offset == 0 (and no q_offset_dev), no
 *     doc_start and 2..16 query heads per KV head: ONE kernel that reads q, k, v, o, d_o once and
 *     produces dq, dk, dv and the dsinks terms from five matrix products per (query tile, key tile)
 *     pair (`_attn_bwd`'s own five dots, attention_kernel.py:199-217), the row statistics formed
 *     on the way, followed by a small kernel that adds the two fp32 shares of the key tiles on the
 *     seams between workgroups and reduces dsinks; `delta` holds those shares and the dsinks
 *     partial sums.  Same values as steps 1-3 up to the order of the fp32 sums (differences in
 *     the last bf16 bit, and of the rare P or dS value that rounds to the other bf16 neighbour
 *     because the dK/dV kernels of steps 1-3 subtract lse inside the matrix product);
 *   - everything else: the dQ kernel computes delta and lse*log2(e) for its own rows (no
 *     separate pass over O and dO), stores them in `delta`, and the dSinks and dK/dV kernels
 *     follow: the same bits as steps 1-3 called one after the other.
 * Both routes are free of atomics and bit-reproducible from run to run.
 * Reads q,k,v,sinks,o,d_o,lse,seqlens,doc_start; writes dq,dk,dv,dsinks,delta.
 */
int gptoss_attn_bwd(const gptoss_attn_params *params, void *stream);

/*
 * The whole backward without any workspace from the caller and without any allocation: a variant
 * of gptoss_attn_bwd whose scratch (the row statistics -rowsum(dO*O) and lse*log2(e)) is an array
 * of GPTOSS_ATTN_STATIC_SCRATCH_BYTES that is part of the library's device image.  It has no
 * counterpart in the reference (whose backward allocates `delta` and zero-filled dk/dv/dsinks with
 * torch, attention_kernel.py:296-303); it is for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  `params->delta` is ignored (may be
 * NULL); inputs and outputs are still the caller's.  Problems with B*H*Sq above 2 097 152 rows are
 * refused with GPTOSS_ATTN_ERR_WORKSPACE before anything is launched.  Key blocks are never cut
 * into slices here (that needs a large scratch), so short full-causal bf16 problems run slower than
 * through gptoss_attn_bwd and their dK/dV may differ from it in the last bit (another summation
 * order); sliding-window layers take the same single-pass kernel, but each workgroup walks two
 * query tiles past its chunk instead of exchanging fp32 shares of the seam tiles (no room for
 * them), so dK/dV of those tiles may differ in the last bit as well; dQ and dSinks are
 * bit-identical.  Every call on one GPU uses that GPU's single array:
 * calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not, and
 * nothing needs clearing between calls (every value read was written earlier in the same call).
 * The array stays resident on every GPU the library has run on until the process ends.
 */
int gptoss_attn_bwd_static(const gptoss_attn_params *params, void *stream);

/* GPTOSS_ATTN_STATIC_SCRATCH_BYTES of the loaded library.  Host-only. */
size_t gptoss_attn_static_scratch_bytes(void);

/*
 * Measurement aid with no counterpart in the reference and no part in the attention path: launches a
 * loop of nothing but bf16 MFMAs (v_mfma_f32_32x32x16_bf16, two wavefronts per SIMD on every compute
 * unit, `iters` passes of 16 MFMAs per wavefront) whose operands are read once from `operands`
 * (`operand_bytes` >= 16, 16-byte aligned device memory, reused cyclically).  A benchmark times it on the
 * kind of data the attention kernels see to learn what the matrix pipes sustain under the part's power
 * limit (the clock under such a loop depends on how many operand bits toggle).  `sink` receives one float
 * per thread (at least 512 * compute units floats, `sink_floats` says how many there are).  Returns the
 * number of MFMA instructions the launch executes (each 32*32*16*2 FLOP), or a negative value: a
 * GPTOSS_ATTN_ERR_* code for bad arguments, -1000 - hipError_t for a failed launch.
 */
int64_t gptoss_attn_mfma_rate_probe(const void *operands, size_t operand_bytes, int iters, float *sink, size_t sink_floats,
                                    void *stream);

/*
 * Second measurement aid, likewise without counterpart in the reference and outside the attention path: runs a
 * synthetic instruction stream with the instruction mix of one of the attention kernels (operands in registers,
 * all zero, so the part's power limit plays no part), one workgroup per compute unit with `waves_per_simd`
 * (1 to 3) wavefronts per SIMD, `iters` passes of 48 MFMAs per wavefront.  `mix`: 0 = MFMAs only, 1 = the forward's
 * mix with every MFMA followed by its share of the vector work, 2 = the forward's work in the order a compiler
 * gives a tile (MFMAs in clumps, the softmax between them), 3 / 4 = the same two for the dQ kernel, 5 = the
 * dK/dV kernel's mix, uniform.  A benchmark times the launches against mix 0 to learn how many matrix-pipe cycles
 * per MFMA such a kernel needs at best on this part.  `sink`: one float per thread (at least 256 * waves_per_simd *
 * compute units).  Returns the number of MFMA instructions the launch executes, or a negative value as for
 * gptoss_attn_mfma_rate_probe.
 */
int64_t gptoss_attn_stream_probe(int mix, int waves_per_simd, int iters, float *sink, size_t sink_floats, void *stream);

/*
 * Host-only argument check used by every entry point; `need_bwd` != 0 also
 * requires the backward tensors.  Callable without a GPU.
 */
int gptoss_attn_validate(const gptoss_attn_params *params, int need_bwd);

#ifdef __cplusplus
}
#endif
#endif /* GPTOSS_ATTN_H */
