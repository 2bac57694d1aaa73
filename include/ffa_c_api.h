/*
 * ffa_c_api.h -- C ABI of the MI355X (gfx950) decode-attention engine.
 *
 * Drop-in boundary for the decode step of szeighami/FastForwardAttention.  Every entry
 * point names the reference interface it replaces (file:line in the reference tree).
 * Plain C: pointers, ints and floats only; no torch types, no C++ templates.
 *
 * Conventions
 *   - all data pointers are DEVICE pointers on the current HIP device, 16-byte aligned;
 *   - fp16 is passed as uint16_t bit patterns (the reference does the same:
 *     attention.cu:1534, torch_ffa_api.cpp:124-126);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream, which is
 *     what the reference always uses: attention.cu:1504);
 *   - the library never allocates: caches, outputs and the workspace belong to the caller;
 *   - every function returns an ffa_status (0 = FFA_OK) and never throws, aborts or
 *     prints.  The reference prints and continues (attention.cu:1444-1451, :1529).
 *
 * Layouts (fixed by the reference, attention.cu:1556-1609)
 *   k_cache [B, H, Dh/x, Lmax, x]   x = 16 / sizeof(T)  (8 for fp16, 4 for fp32)
 *   v_cache [B, H, Lmax, Dh]
 *   q, k, v, out  [B, H, Dh] contiguous
 */
#ifndef FFA_C_API_H
#define FFA_C_API_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FFA_API_VERSION 1

typedef enum ffa_status {
    FFA_OK = 0,
    FFA_ERR_NULL_POINTER = 1,   /* a required pointer is NULL                                */
    FFA_ERR_DTYPE = 2,          /* precision is neither 16 nor 32                            */
    FFA_ERR_HEAD_DIM = 3,       /* Dh not one of 64, 80, 128, 256                            */
    FFA_ERR_SHAPE = 4,          /* B, H, L or Lmax not positive, or L > Lmax                 */
    FFA_ERR_TIMESTEP = 5,       /* t outside [0, Lmax)                                       */
    FFA_ERR_ALIGNMENT = 6,      /* a pointer is not 16-byte aligned                          */
    FFA_ERR_WORKSPACE = 7,      /* workspace NULL/too small for the chosen plan              */
    FFA_ERR_PLAN = 8,           /* malformed launch plan                                     */
    FFA_ERR_TOO_LONG = 9,       /* t+1 scores do not fit the LDS of an FFA_LAUNCH_WORKGROUP plan */
    FFA_ERR_PROB_THRESH = 10,   /* p is negative or NaN                                      */
    FFA_ERR_LAUNCH = 11,        /* the HIP runtime refused the launch                        */
    FFA_ERR_NO_DEVICE = 12,     /* no usable gfx950 device / HIP runtime error               */
    FFA_ERR_SCRATCH_LIMIT = 13, /* ffa_attention_static_scratch: the plan needs more scratch */
                                /* than FFA_STATIC_SCRATCH_BYTES                             */
    FFA_ERR_TRANSFORM = 14,     /* rotary_embedding_dim odd, negative or > head_dim, or a    */
                                /* bias pointer not 16-byte aligned                          */
    FFA_ERR_BEAM = 15           /* beam indirection: NULL or misaligned table, beam_width    */
                                /* < 1 or not a divisor of batch_size, or a group too large   */
} ffa_status;

/* precision codes: the same integers the reference passes to get_launch_params
 * (torch_ffa_api.cpp:174). */
#define FFA_PRECISION_F16 16
#define FFA_PRECISION_F32 32
/* bfloat16 (1-8-7), accepted by ffa_attention_ex, ffa_attention_diag and
 * ffa_attention_static_scratch (and by the planner, which plans it like fp16).  The reference
 * carries a bf16 build (ENABLE_BF16, decoder_masked_multihead_attention_utils.h:44-125) that it
 * never enables. */
#define FFA_PRECISION_BF16 0xBF16

/* Launch kinds. */
#define FFA_LAUNCH_WORKGROUP 0  /* one workgroup per (batch, head); scores staged in LDS;   */
                                /* any p >= 0.  The analogue of the reference's launch.     */
#define FFA_LAUNCH_SPLIT 1      /* online-softmax kernel, p == 0 only: whole_heads pairs    */
                                /* with one workgroup each, the others split over n_splits  */
                                /* workgroups whose partials the last arriver combines      */
#define FFA_LAUNCH_TWO_PASS 2   /* any p >= 0, any length: a scores kernel (K stream, raw   */
                                /* scores to the workspace) then a weights x V kernel that  */
                                /* reads only surviving rows; n_splits pieces per pair      */

/* How the partial (max, sum, acc[Dh]) results of a split launch are merged. */
#define FFA_COMBINE_FUSED 0     /* by the last workgroup of each (batch, head) to arrive     */
#define FFA_COMBINE_KERNEL 1    /* by a second, small kernel on the same stream              */

/* Replaces the (tpb, tpv, tpk) triple of kernel_launch_utils.h:135-180. */
typedef struct ffa_launch_plan {
    int32_t kind;             /* FFA_LAUNCH_*                                              */
    int32_t waves_per_wg;     /* wave64 wavefronts per workgroup: 1, 2, 4, 8 or 16; also   */
                              /* 3, 5, 6, 7 in FFA_LAUNCH_SPLIT plans with one lane per key */
    int32_t threads_per_key;  /* lanes cooperating on one key's q.k: 1, or 2 / 4 in        */
                              /* FFA_LAUNCH_SPLIT plans with 4 or 8 waves (head dims 64,   */
                              /* 128 and, for 4 lanes, 256 in fp16 / 128 in fp32)          */
    int32_t keys_per_wave;    /* 64 / threads_per_key: keys a wavefront handles per tile   */
    int32_t n_splits;         /* workgroups per (batch, head); 1 for FFA_LAUNCH_WORKGROUP  */
    int32_t tiles_per_split;  /* 64-key blocks each split walks (whatever the tile size)   */
    int32_t combine;          /* FFA_COMBINE_*: how split partials are merged              */
    int32_t whole_heads;      /* FFA_LAUNCH_SPLIT: the first whole_heads (batch, head)     */
                              /* pairs get ONE workgroup each (no cross-workgroup merge);  */
                              /* only the remaining pairs are split n_splits ways          */
} ffa_launch_plan;

int ffa_api_version(void);
const char* ffa_status_string(int status);

/* Number of compute units of the current device (256 on MI355X); <= 0 if none. */
int ffa_device_compute_units(void);

/*
 * Launch planner.  Replaces get_launch_params (kernel_launch_utils.h:135-180).
 *   precision  16 | 32;  t = number of cached keys at the step being planned (the
 *   reference plans once on the prompt length, torch_ffa_api.cpp:176; this planner is
 *   cheap enough to be called per step);  prob_thresh: the p the step will use;
 *   use_default_kernel_launch != 0 -> one workgroup per (batch, head), workgroup size by
 *   sequence length, like the FasterTransformer table at kernel_launch_utils.h:137-154;
 *   == 0 -> tuned plan for `compute_units` CUs (pass 0 to query the current device): rules
 *   derived from measurements, overridden at the shapes of a sweep on the device where the
 *   sweep found a faster launch (csrc/ffa_plan_table.inc, `python bench.py --sweep-plans`).
 */
int ffa_plan_launch(int precision, int batch_size, int head_num, int head_dim,
                    int t, float prob_thresh, int use_default_kernel_launch,
                    int compute_units, ffa_launch_plan* plan);

/* The same planner with its table of measured overrides ignored: what the rules alone would
 * launch.  The tuned planner is rules + a table generated by a sweep on the device (the
 * working analogue of the fitted time model at kernel_launch_utils.h:85-132); this entry is
 * what that sweep compares its candidates against. */
int ffa_plan_launch_rules(int precision, int batch_size, int head_num, int head_dim,
                          int t, float prob_thresh, int use_default_kernel_launch,
                          int compute_units, ffa_launch_plan* plan);

/* Where ffa_plan_launch takes the tuned plan of a problem from: 0 = the rules, 1 = a row of the
 * table measured at the BASELINE shapes (exact match), 2 = the nearest row of the measured grid
 * (csrc/ffa_plan_grid.inc, `python bench.py --sweep-plans grid`).  Negative = bad arguments.  No
 * counterpart in the reference, whose fitted model (kernel_launch_utils.h:85-132) has one source. */
int ffa_plan_source(int precision, int batch_size, int head_num, int head_dim, int t,
                    float prob_thresh, int compute_units);

/* Bytes of device workspace sufficient for ANY plan this library produces for the
 * given problem (arrival counters, split partials, two-pass scores). */
size_t ffa_workspace_bytes(int batch_size, int head_num, int head_dim, int max_seq_len);

/* Zero a workspace (what matters are the arrival counters at its head; the buffer may be of
 * ffa_workspace_bytes() bytes or sized for one plan).  Call once before first use, and again after any launch
 * on the workspace that failed or was aborted: a launch that dies half-way leaves counters
 * non-zero, and later launches would then never merge their pieces.
 * One workspace serves one stream at a time: two launches that overlap on the same
 * workspace race on its counters and partials. */
int ffa_workspace_init(void* workspace, size_t workspace_bytes, void* stream);

/*
 * Cache construction.  Replaces invokeTranspose4dBatchMajor<T>
 * (torch_ffa_api.cpp:14-47; attention.cu:1611-1689) -- same argument order.
 *   k_dst [B,H,Dh/x,Lmax,x], v_dst [B,H,Lmax,Dh]  <-  k_src, v_src [B,H,L,Dh].
 * Slots l >= seq_len are left untouched, as in the reference.
 */
int ffa_init_cache_f16(uint16_t* k_dst, uint16_t* v_dst, const uint16_t* k_src,
                       const uint16_t* v_src, int batch_size, int seq_len, int max_seq_len,
                       int head_dim, int head_num, void* stream);
int ffa_init_cache_f32(float* k_dst, float* v_dst, const float* k_src, const float* v_src,
                       int batch_size, int seq_len, int max_seq_len, int head_dim,
                       int head_num, void* stream);

/*
 * One decode-attention step.  Replaces call_attention<T> (c_ffa_api.h:10-14;
 * attention.cu:1512-1554) and do_attention<T> (c_ffa_api.h:17-20): appends k, v at
 * cache slot t and writes out[b,h,:] = sum_i P_i V_i over keys first_key .. t.
 *   seq_lengths (device int[B]) may be NULL.  With right_or_no_padding != 0 it is the
 *   per-sample slot/length that replaces t (attention.cu:809-811; every entry must be
 *   <= t); with right_or_no_padding == 0 it is the index of the first real key of a
 *   left-padded sample (attention.cu:814-817).
 *   prob_thresh == 0: exact attention.  prob_thresh > 0: the reference's pruning rule
 *   (attention.cu:1184-1191): key i < t is dropped iff leq(T(e_i*inv), T(p*inv)).
 *   plan: NULL -> planned internally as ffa_plan_launch(..., use_default = 0).
 *   workspace: required unless the plan is FFA_LAUNCH_WORKGROUP.
 */
int ffa_attention_f16(int batch_size, int head_num, int head_dim, int max_seq_len,
                      float softmax_scale, int t, const uint16_t* q, const uint16_t* k,
                      const uint16_t* v, uint16_t* k_cache, uint16_t* v_cache, uint16_t* out,
                      const int* seq_lengths, float prob_thresh, const ffa_launch_plan* plan,
                      int right_or_no_padding, void* workspace, size_t workspace_bytes,
                      void* stream);
int ffa_attention_f32(int batch_size, int head_num, int head_dim, int max_seq_len,
                      float softmax_scale, int t, const float* q, const float* k,
                      const float* v, float* k_cache, float* v_cache, float* out,
                      const int* seq_lengths, float prob_thresh, const ffa_launch_plan* plan,
                      int right_or_no_padding, void* workspace, size_t workspace_bytes,
                      void* stream);

/*
 * Same step with pruning diagnostics (no counterpart in the reference, which never
 * reports what it skipped; needed to report the fraction of keys skipped):
 *   kept_count  device uint32[B*H] or NULL: number of cached keys i < t whose V row was
 *               read (overwritten, not accumulated);
 *   skip_mask   device uint8[B*H*Lmax] or NULL: 1 where key i < t was dropped.
 * The exact split kernel keeps no diagnostics: a NULL plan is planned as for a pruned
 * step, an FFA_LAUNCH_SPLIT plan is rejected with FFA_ERR_PLAN.  With prob_thresh == 0 only
 * masked (left-padding) keys count as dropped and kept_count[b,h] = t - first_key.
 */
int ffa_attention_diag(int precision, int batch_size, int head_num, int head_dim,
                       int max_seq_len, float softmax_scale, int t, const void* q,
                       const void* k, const void* v, void* k_cache, void* v_cache, void* out,
                       const int* seq_lengths, float prob_thresh, const ffa_launch_plan* plan,
                       int right_or_no_padding, void* workspace, size_t workspace_bytes,
                       uint32_t* kept_count, uint8_t* skip_mask, void* stream);

/*
 * The decode step with the FasterTransformer features that the reference's kernel carries but
 * its host code switches off (attention.cu:1472-1483): q/k/v bias (attention.cu:856-873,
 * :1157-1158, :1242), rotary position embedding of q and k (attention.cu:874-882;
 * decoder_masked_multihead_attention_utils.h:1137-1160), the beam-search cache indirection
 * and a bf16 element type.
 *   precision  FFA_PRECISION_F16 | FFA_PRECISION_F32 | FFA_PRECISION_BF16 (bf16 caches are built
 *              with ffa_init_cache_f16: cache construction only moves 16-byte chunks);
 *   transform  NULL = none (then the call equals ffa_attention_f16 / _f32).  Otherwise, before
 *              the step and in this order: q += q_bias, k += k_bias, v += v_bias (device
 *              [H, Dh] arrays of the element type, each may be NULL); then, if
 *              rotary_embedding_dim > 0 (even, <= head_dim), the pairs (2i, 2i+1) below that
 *              dimension of q and k are rotated by pos / base^(2i / rotary_embedding_dim)
 *              (GPT-J's pairing), evaluated in double precision and rounded once to the
 *              element type.  pos is the number of
 *              real tokens before the new one: t, or seq_lengths[b] with right padding, or
 *              t - seq_lengths[b] with left padding (the reference rotates by t alone and so
 *              supports no padded batch, attention.cu:879).  The transformed k and v are what
 *              the caches receive.  It runs inside the decode launch (no kernel of its own,
 *              no workspace): one wave per workgroup computes the angles, every wave rotates
 *              its own copy of q, the wave that appends the token also k and v.
 *   beams      NULL = none.  Otherwise beam-search cache indirection (attention.cu:779-793,
 *              :1003, :1024-1033, :1143, :1195-1202; the reference's host code passes nullptr
 *              and beam_width 1, attention.cu:1477-1479): sample b is beam b % beam_width of
 *              group b / beam_width, and its cached key i < t is read from the caches of
 *              sample (b - b % beam_width) + cache_indir[b * max_seq_len + i] instead of its own;
 *              the new token is appended to the sample's own caches as always.  A search then
 *              re-parents beams by permuting rows of this small table instead of copying
 *              caches.  Entries outside [0, beam_width) are clamped into that range.  All
 *              beams of a group must be at the same length (same t, same seq_lengths entry):
 *              a beam's slot t is written in the launch in which its siblings read the slots
 *              below theirs.  batch_size must be a multiple of beam_width and
 *              beam_width * head_num * max_seq_len must stay below 2^31 (FFA_ERR_BEAM).
 *              Every launch plan takes an indirection.
 */
typedef struct ffa_token_transform {
    const void* q_bias;
    const void* k_bias;
    const void* v_bias;
    int32_t rotary_embedding_dim; /* 0 = no rotary embedding                                   */
    float rotary_base;            /* 10000 in the reference (utils.h:1139); <= 0 selects that  */
} ffa_token_transform;

typedef struct ffa_beam_indirection {
    const int32_t* cache_indir; /* device, [batch_size, max_seq_len]: source beam of each key */
    int32_t beam_width;         /* samples per group, >= 1                                    */
} ffa_beam_indirection;

int ffa_attention_ex(int precision, int batch_size, int head_num, int head_dim, int max_seq_len,
                     float softmax_scale, int t, const void* q, const void* k, const void* v,
                     void* k_cache, void* v_cache, void* out, const int* seq_lengths,
                     float prob_thresh, const ffa_launch_plan* plan, int right_or_no_padding,
                     const ffa_token_transform* transform, const ffa_beam_indirection* beams,
                     void* workspace, size_t workspace_bytes, void* stream);

/*
 * The same step for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  It takes no workspace: arrival counters, split partials and two-pass scores
 * live in a static device array of FFA_STATIC_SCRATCH_BYTES inside the library (one copy per
 * GPU, held until the process ends), and the call allocates and frees nothing.
 *   - a plan (given, or chosen internally when plan == NULL) whose workspace need exceeds
 *     FFA_STATIC_SCRATCH_BYTES is refused with FFA_ERR_SCRATCH_LIMIT before anything is
 *     launched; FFA_LAUNCH_WORKGROUP plans need none;
 *   - every call on a GPU shares that GPU's array: calls that overlap on one GPU (two
 *     streams, two host threads) race; calls on one stream are ordered and safe;
 *   - the arrival counters of the call's (batch, head) pairs are cleared by a small kernel
 *     on `stream` ahead of the decode kernel.
 * Arguments as ffa_attention_ex (transform and beams may be NULL), without the workspace.
 */
#define FFA_STATIC_SCRATCH_BYTES (4u << 20)
int ffa_attention_static_scratch(int precision, int batch_size, int head_num, int head_dim,
                                  int max_seq_len, float softmax_scale, int t, const void* q,
                                  const void* k, const void* v, void* k_cache, void* v_cache,
                                  void* out, const int* seq_lengths, float prob_thresh,
                                  const ffa_launch_plan* plan, int right_or_no_padding,
                                  const ffa_token_transform* transform,
                                  const ffa_beam_indirection* beams, void* stream);

/*
 * Measurement aid, no counterpart in the reference: the load floor of an FFA_LAUNCH_SPLIT plan
 * with one lane per key and 2, 4 or 8 waves.  Launches the grid, the workgroups and the tile walk
 * of the decode kernel for this plan and issues every 16-byte load of K and V that the step would
 * issue (cached keys 0 .. t-1), the same number in flight per wave -- no arithmetic, no merge, no
 * output.  Its duration is what the memory system gives this launch shape; bench.py reports the
 * decode kernels against it.  `sink`: 16 bytes of device memory, 16-byte aligned (the probe stores
 * to it only if the XOR of everything it loaded equals one fixed value); the caches are only read.
 */
int ffa_load_floor(int precision, int batch_size, int head_num, int head_dim, int max_seq_len, int t,
                   const void* k_cache, const void* v_cache, const int* seq_lengths,
                   int right_or_no_padding, const ffa_launch_plan* plan, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FFA_C_API_H */
