/*
 * tinyllm_hybrid.h — C ABI of the layer-list engine ("hybrid engine"): decoder-only models whose layers are
 * described one by one (a token mixer of some kind, an optional feed-forward, one shared pre-norm), with
 * unquantised bf16 or fp32 weights and a float32 residual stream.
 *
 * Where the Qwen3 engine (tinyllm_engine.h) is one fixed layer shape issued as 5 fused W4 kernels, this engine
 * walks a list of layer descriptions.  Mixer kinds so far:
 *
 *   TL_MIX_ATTENTION   grouped-query softmax attention over the paged K/V pool.  Options per layer: rotary
 *                      positions on the first rot_dims dimensions of each head (adjacent pairs), unit-RMS
 *                      normalisation of q and k after the rotation, a score scale, a "sink" (one is added to the
 *                      softmax denominator: a key of score 0 without a value), a sigmoid output gate.
 *                      Query/key width and value width of a head are independent.
 *   TL_MIX_DELTA       gated delta rule: a [key_dim, value_dim] float32 state per head that decays, is corrected
 *                      towards the new value along the new key and is read with the query; q/k/v pass a short
 *                      causal depthwise convolution + SiLU first.  The state and the convolution's last inputs
 *                      live in one state slot per sequence.
 *
 * A contiguous range of layers may be repeated ("loop"): each pass has its own K/V pages / state slots, and is
 * entered through a [width, 2 width] projection of the running stream beside the embedding output plus a per-pass
 * offset vector.
 *
 * One step function serves prefill, decode and any mixture: tl_hybrid_step takes chunks of token ids for several
 * sequence slots (a chunk of one token is a decode step), runs them as one packed batch of rows and returns the
 * logits of the rows asked for.  Row-wise work (norms, projections, feed-forward) runs once over the packed rows;
 * attention and the recurrences run per sequence from what earlier steps left in the pages and state slots.
 *
 * Float32 throughout: residual stream, norms, rotary angles, attention scores / weights, decays, gates of the
 * recurrence, recurrent state.  With dtype TL_BF16 the matrices, the activations entering a matrix product and
 * the K/V pages are bfloat16 (float32 accumulation); with TL_F32 everything is float32 (fp32 MFMA, no reduced mode).
 *
 * All functions return 0 / negative tl_status; message via tl_hybrid_last_error().  *_dev = device pointers.
 */
#ifndef TINYLLM_HYBRID_H
#define TINYLLM_HYBRID_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tl_hybrid tl_hybrid;

enum { TL_MIX_ATTENTION = 0, TL_MIX_DELTA = 1 };
enum { TL_HY_F32 = 0, TL_HY_BF16 = 2 }; /* the values of tl_dtype in tinyllm_hip.h */

/* One layer.  Matrices are [out, in] row-major in the engine's dtype; vectors are float32.
 * w_in: every projection that reads the normed input, rows concatenated in this order:
 *   attention: q (heads*dim) | k (kv_heads*dim) | v (kv_heads*vdim) | gate (heads*vdim, if gated) | up (ff, if ff > 0)
 *   delta:     q (kv_heads*dim) | k (kv_heads*dim) | v (heads*vdim) | gate (heads*vdim) | a (heads) | b (heads) | up (ff)
 * w_out: [width, heads*vdim + ff]: the mixer's output projection beside the feed-forward's down projection, so
 *   one product yields mixer(h) + ff(h). */
typedef struct tl_hybrid_layer {
    int kind;
    int heads, kv_heads, dim, vdim;
    int ff;                 /* 0: no feed-forward */
    int ff_act;             /* 0 exact (erf) GELU, 1 tanh GELU, 2 SiLU */
    const void *w_in_dev, *w_out_dev;
    const float *norm_dev;  /* [width] pre-norm weight */
    float norm_offset;      /* weight is applied as (norm_offset + w): 1 for weights stored around zero */
    /* attention */
    int rot_dims;           /* 0: no rotary positions */
    float rot_base;
    float scale;
    int qk_unit_rms;        /* q and k divided by their RMS over dim after the rotation */
    int sink;               /* softmax denominator += 1 */
    int gated;              /* output * sigmoid(gate) */
    /* delta */
    int conv_taps;
    const float *conv_dev;  /* [2*kv_heads*dim + heads*vdim, taps], last tap = current token */
    const float *a_log_dev, *dt_bias_dev; /* [heads] */
    const float *out_norm_dev;            /* [vdim] */
    float unit_eps;         /* q, k -> x / sqrt(sum x^2 + unit_eps) */
} tl_hybrid_layer;

typedef struct tl_hybrid_config {
    int dtype;              /* TL_HY_BF16 or TL_HY_F32 */
    int width, vocab, num_layers;
    float norm_eps, residual_mult;
    int parallel_block;     /* 1: x += m * (mixer(h) + ff(h)) with one norm (the only form so far) */
    int loop_start, loop_stop, loop_times; /* loop_times <= 1 or start == stop: no loop */
    const void *loop_in_dev;    /* [width, 2*width], stream first */
    const float *loop_step_dev; /* [loop_times, width] */
    const void *embed_dev;      /* [vocab, width] */
    const float *final_norm_dev;
    float final_norm_offset;
    const void *head_dev;       /* [vocab, width] */
    int page_size, num_pages, max_slots, max_pages_per_seq, max_rows;
} tl_hybrid_config;

typedef struct tl_hybrid_stats {
    int pages_in_use, pages_free, peak_pages_in_use;
    long page_allocations, reused_page_allocations;
    long steps, rows, slot_begins, reused_slot_begins;
    size_t kv_bytes, state_bytes, workspace_bytes;
    int layer_runs;
    long graph_captures, graph_replays;
} tl_hybrid_stats;

const char *tl_hybrid_last_error(void);

/* Weight memory is borrowed and must outlive the engine.  stream: the hipStream_t all work is issued on; NULL makes
 * the engine create and own one. */
int tl_hybrid_create(const tl_hybrid_config *cfg, const tl_hybrid_layer *layers, void *stream, tl_hybrid **out);
void tl_hybrid_destroy(tl_hybrid *e);
int tl_hybrid_synchronize(tl_hybrid *e);

/* begin: claim a free slot, context 0, recurrent state and convolution inputs zeroed.  release: pages back to the
 * free list; the slot may be claimed again. */
int tl_hybrid_begin(tl_hybrid *e, int slot);
int tl_hybrid_release(tl_hybrid *e, int slot);
int tl_hybrid_context_len(const tl_hybrid *e, int slot);
/* The sequence of the live slot `src` changes hands to the free slot `dst`: block-table row, context length and pending
 * token move, K/V pages stay; the recurrent state and convolution inputs of every delta layer run are copied. */
int tl_hybrid_move(tl_hybrid *e, int src, int dst);

/* One packed step.  tokens = the chunks back to back, lens[i] tokens for slots[i] (distinct, live) at positions
 * [context_i, context_i + lens[i]); sum(lens) <= max_rows.  want_rows[j] = index into the packed rows whose logits
 * are computed: row j of the logits buffer.  All-or-nothing: everything is checked and pages are reserved before
 * anything runs.  Enqueues only; the logits are read with tl_hybrid_copy_logits / tl_hybrid_read_argmax. */
int tl_hybrid_step(tl_hybrid *e, int n_seqs, const int *slots, const int32_t *tokens, const int *lens, int n_want,
                   const int *want_rows);

/* Greedy decode of the live slots listed: each slot's pending token (tl_hybrid_set_token, or the argmax of its last
 * wanted row) is fed as a one-token chunk; the argmax of its logits becomes the new pending token.  `steps` steps are
 * enqueued without host involvement between them (captured in a hipGraph per batch shape where use_graph != 0). */
int tl_hybrid_decode(tl_hybrid *e, int n_seqs, const int *slots, int steps, int use_graph);
int tl_hybrid_set_token(tl_hybrid *e, int slot, int32_t token);
/* Pending token of each listed slot after synchronising. */
int tl_hybrid_read_pending(tl_hybrid *e, int n, const int *slots, int32_t *out);

/* Stream-ordered copy of the first `rows` rows of the latest logits [rows, vocab] float32 to device or host memory;
 * the host form synchronises. */
int tl_hybrid_copy_logits(tl_hybrid *e, void *dst_dev, int rows);
int tl_hybrid_read_logits(tl_hybrid *e, float *dst_host, int rows);
/* argmax of the first `rows` logits rows; synchronises. */
int tl_hybrid_read_argmax(tl_hybrid *e, int rows, int32_t *out);

/* Test aid: the residual stream after layer run `run` of the latest step ([rows, width] float32) is kept when
 * tracing is on (one extra copy per layer run). */
int tl_hybrid_set_trace(tl_hybrid *e, int on);
int tl_hybrid_read_trace(tl_hybrid *e, int run, float *dst_host, int rows);

int tl_hybrid_get_stats(const tl_hybrid *e, tl_hybrid_stats *out);

/* Kernel-level entry points on caller buffers (tests, microbenchmarks).  dtype as in the config. */
int tl_hybrid_linear(int dtype, const void *a_dev, int lda, const void *w_dev, float *out_dev, int ldc, int M, int N, int K,
                     int force_kernel /* 0 by shape, 1 row kernel, 2 64-wide tile kernel, 3 256-wide tile GEMM (bfloat16) */, void *stream);

#ifdef __cplusplus
}
#endif
#endif
