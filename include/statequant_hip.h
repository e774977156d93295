/* C ABI of libsqhip.so: the packed recurrent-state decode step on one MI355X (gfx950).
 *
 * Every entry point takes plain device pointers, element strides and sizes; nothing here allocates, frees, retains
 * a pointer or synchronizes.  Work is enqueued on the HIP stream passed as `stream` (a hipStream_t; NULL = the null
 * stream), so calls are safe under HIP graph capture.  Return value: 0 on success, otherwise a negative SQ_E_* code
 * (sq_strerror() names it; sq_last_error() gives the detail of the last failure on the calling thread).
 *
 * The entry points replace the Triton launch sites of the reference (paths relative to
 * /root/reference/src/statequant/kernels/):
 *   sq_gdn_step     _fused_triton.py:48 `_fused_step`, launched from fold.py:400-408 (lockstep) and
 *                   slots.py:178-187 (slot-addressed)
 *   sq_kda_step     _kda_triton.py:38 `_kda_step`, launched from kda.py:192-205
 *   sq_mamba2_step  _mamba2_triton.py:48 `_m2_step`, launched from mamba2.py:223-241
 *   sq_pack_vk      fold.py:123-147 `pack_vk` / slots.py:236-252 `write` (torch in the reference)
 *   sq_read         slots.py:210-233, kda.py:351-372 `read` (torch in the reference)
 *   sq_gga_step     _gga_triton.py:207 `_gga_step` + :300 `_gga_advance`, launched from
 *                   ../integrations/vllm_gga.py:240-253 (`GGAPacked.step`)
 *   sq_gga_store    _gga_triton.py:314 `_gga_store` (vllm_gga.py:305-318, `GGAPacked.write`)
 *   sq_gga_load     _gga_triton.py:331 `_gga_load` (vllm_gga.py:255-267, `GGAPacked.stored`)
 * The argument convention is the reference's (_fold_triton.py:30-36): every per-sequence tensor comes as a base
 * pointer plus its per-sequence stride IN ELEMENTS of that tensor's type; batch row b works on sequence idx[b]
 * (idx == NULL: sequence b); rows with idx[b] <= 0 are padding: their output row is zeroed, nothing else is touched.
 */
#ifndef STATEQUANT_HIP_H
#define STATEQUANT_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SQ_ABI_VERSION 6

enum { SQ_F32 = 0, SQ_BF16 = 1, SQ_F16 = 2 };                /* dtype codes of float tensors */

enum {
    SQ_OK = 0,
    SQ_E_ARG = -1,          /* a null pointer, bad stride / alignment or inconsistent sizes */
    SQ_E_UNSUPPORTED = -2,  /* a (bits, axis, group, d_k, d_v, m, buffer) combination no kernel is built for */
    SQ_E_LAUNCH = -3        /* the HIP runtime refused the launch (sq_last_error() holds hipGetErrorString) */
};

/* The stored state and decode buffer of a set of sequences (slots.py:9-22 for the field meanings and shapes).
 * S     codes: int8 [hv, dv, dk] (bits 8) or uint8 [hv, dv, dk/2] (bits 4, byte j = (c[2j]+8) | (c[2j+1]+8) << 4);
 *       the unquantized control: bf16 (bits 16) or fp32 (bits 32) [hv, dv, dk] (fold.py:128-129, slots.py:55-56)
 * SC    fp16 scales [hv, dv, ceil(dk/group)] (key-axis groups) or [hv, dv/group, dk] (value-axis groups);
 *       ignored (may be NULL) for the unquantized control
 * Every stride s* counts elements of its own tensor per sequence (sS: codes bytes, or bf16 / fp32 elements).
 * KB    buffered keys [hk, m, dk], int8 (buffer_bits 8) or bf16 (16);  KBS fp16 [hk, m] (int8 buffer only)
 * UB    buffered delta values [hv, m, dv], int8 or bf16;               UBS fp16 [hv, m] (int8 buffer only)
 * GB    fp32 cumulative log decay of each buffered token: [hv, m] (GDN, Mamba2) or [hv, m, dk] (KDA)
 * GCUR  fp32 running log decay since the last fold: [hv] or [hv, dk] (KDA)
 * NPTR  int32 buffer fill counter, one copy per value head: element h of a sequence belongs to head h */
typedef struct sq_state {
    void* S;        int64_t sS;
    void* SC;       int64_t sSC;
    void* KB;       int64_t sKB;
    void* KBS;      int64_t sKBS;
    void* UB;       int64_t sUB;
    void* UBS;      int64_t sUBS;
    float* GB;      int64_t sGB;
    float* GCUR;    int64_t sGC;
    int32_t* NPTR;  int64_t sN;
} sq_state;

/* Layer geometry and storage format (fold.py:91-104 `packed_format`, slots.py:53-74). */
typedef struct sq_layout {
    int32_t bits;         /* 4 or 8: codes; 16 / 32: the state kept as bf16 / fp32, no scales (axis_k, group ignored) */
    int32_t axis_k;       /* 1: scale groups along d_k; 0: along d_v (group rows of one key column share a scale) */
    int32_t group;        /* scale group length, a power of two (value-axis: must divide d_v; built for 16, 32, 64) */
    int32_t buffer_bits;  /* 8 (int8 + fp16 scale per vector) or 16 (bf16) */
    int32_t m;            /* buffer length, a power of two */
    int32_t hv, hk;       /* value heads, key heads (groups); hv % hk == 0 */
    int32_t dk, dv;       /* head dims */
} sq_layout;

/* One Gated DeltaNet decode token per batch row (fold.py:381-408, slots.py:124-187).
 * q, k   [rows, hk, dk] (qk_per_key_head = 1) or [rows, hv, dk] (0), raw; l2-normalised in the kernel
 * v      [rows, hv, dv];  out [rows, hv, dv] contiguous
 * gate = 0: g, beta [rows, hv] (log decay, sigmoided beta)
 * gate = 1: a, b [rows, hv], A_log, dt_bias [hv]: g = -exp(A_log) softplus(a + dt_bias), beta = sigmoid(b)
 * Row strides (s_*) are in elements; inner dims are contiguous. */
typedef struct sq_gdn_args {
    sq_state st;
    sq_layout lay;
    int32_t rows;
    const int32_t* idx;
    const void* q;      int64_t s_q;     int32_t q_dtype;
    const void* k;      int64_t s_k;     int32_t k_dtype;
    const void* v;      int64_t s_v;     int32_t v_dtype;
    int32_t qk_per_key_head;
    int32_t gate;
    const void* g;      int64_t s_g;     int32_t g_dtype;
    const void* beta;   int64_t s_beta;  int32_t beta_dtype;
    const void* a;      int64_t s_a;     int32_t a_dtype;
    const void* b;      int64_t s_b;     int32_t b_dtype;
    const void* A_log;  int32_t A_log_dtype;
    const void* dt_bias; int32_t dt_bias_dtype;
    void* out;          int32_t out_dtype;
    float scale;
    /* Optional dispatch order of the batch rows (NULL: the batch order): order[p] is the batch row that position p of
     * the launch works on, a permutation of 0 .. rows-1.  Results do not depend on it.  No counterpart in the
     * reference: a scheduling hint for batches whose sequences fill their buffers on different steps, where the rows
     * that fold on this step keep their workgroups longer and their place in the launch decides when it ends (on the
     * 256-slot int8 step: 38.4 us per launch in batch order, 33.0 with the order of sq_fold_order, 32.2 when all
     * sequences fold together).  sq_fold_order() writes such a list from the counters. */
    const int32_t* order;
} sq_gdn_args;

/* One KDA decode token per batch row (kda.py:192-205, 330-347): per-key-channel log decay g [rows, hv, dk];
 * hk == hv.  q, k [rows, hv, dk], v [rows, hv, dv], beta [rows, hv], out [rows, hv, dv] with row stride s_out. */
typedef struct sq_kda_args {
    sq_state st;
    sq_layout lay;
    int32_t rows;
    const int32_t* idx;
    const void* q;      int64_t s_q;     int32_t q_dtype;
    const void* k;      int64_t s_k;     int32_t k_dtype;
    const void* v;      int64_t s_v;     int32_t v_dtype;
    const void* g;      int64_t s_g;     int32_t g_dtype;
    const void* beta;   int64_t s_beta;  int32_t beta_dtype;
    void* out;          int64_t s_out;   int32_t out_dtype;
    float scale;
    const int32_t* order;   /* optional dispatch order of the rows, as in sq_gdn_args */
} sq_kda_args;

/* One Mamba2 / SSD decode token per batch row (mamba2.py:223-241, 377-396).
 * x [rows, hv, dv], dt [rows, hv] raw, B / C [rows, hk, dk] (hk = groups), A [hv], D / dt_bias [hv] or NULL,
 * out [rows, hv, dv] with row stride s_out.  dt <- dt + dt_bias; softplus (threshold 20) if dt_softplus;
 * clamped to [dt_min, dt_max] if dt_clamp. */
typedef struct sq_mamba2_args {
    sq_state st;
    sq_layout lay;
    int32_t rows;
    const int32_t* idx;
    const void* x;      int64_t s_x;     int32_t x_dtype;
    const void* dt;     int64_t s_dt;    int32_t dt_dtype;
    const void* B;      int64_t s_B;     int32_t B_dtype;
    const void* C;      int64_t s_C;     int32_t C_dtype;
    const void* A;      int32_t A_dtype;
    const void* D;      int32_t D_dtype;
    const void* dt_bias; int32_t dt_bias_dtype;
    int32_t dt_softplus;
    int32_t dt_clamp;   float dt_min, dt_max;
    void* out;          int64_t s_out;   int32_t out_dtype;
    const int32_t* order;   /* optional dispatch order of the rows, as in sq_gdn_args */
} sq_mamba2_args;

/* Store fp32 states in the packed format (fold.py:123-147 `pack_vk`; with idx, GCUR and NPTR given this is
 * slots.py:236-252 `SlotLayout.write`: the states go into sequences idx[b] and those sequences' buffers are emptied).
 * src [rows, hv, dv, dk] value-major fp32, row stride s_src in elements; codes / scales as in sq_state.
 * Uses lay.bits, axis_k, group, hv, dk, dv.  GCUR / NPTR may be NULL (left alone); nptr_copies = counter copies per sequence that are zeroed (the slot
 * layout keeps max(hv, 4), slots.py:13-15; 0 means hv); gcur_per_head = 1 (GDN, Mamba2)
 * or dk (KDA).  Rows with idx[b] <= 0 are skipped. */
typedef struct sq_pack_args {
    sq_layout lay;
    int32_t rows;
    const int32_t* idx;
    const float* src;   int64_t s_src;
    void* S;            int64_t sS;
    void* SC;           int64_t sSC;
    float* GCUR;        int64_t sGC;     int32_t gcur_per_head;
    int32_t* NPTR;      int64_t sN;      int32_t nptr_copies;
} sq_pack_args;

/* The current state of sequences idx[b] as fp32 value-major [rows, hv, dv, dk] (row stride s_out in elements): the
 * stored state advanced across its pending buffer, a_n S_0 + sum_{i<n} (a_n / a_i) u_i k_i^T (slots.py:210-233;
 * kda = 1: decays per key channel, kda.py:351-372).  Nothing is modified.  Rows with idx[b] <= 0 are skipped. */
typedef struct sq_read_args {
    sq_state st;
    sq_layout lay;
    int32_t kda;
    int32_t rows;
    const int32_t* idx;
    float* out;         int64_t s_out;
} sq_read_args;

/* The mixed-width GGA / STEP slot of one layer (../integrations/vllm_gga.py:185-217 `GGAPacked`; byte layout in
 * _gga_triton.py:3-13).  One blob per slot:
 *   bytes 0..15     int32 n (queued pairs), head (ring index of the oldest pair), 2 unused
 *   offs[h]         value head h at its frozen width bits[h]: 16 = fp16 [dk, dv]; 4, 6, 8 = codes [dk, dv*b/8] (u = z +
 *                   qmax, little-endian along dv), row factors fp16 [dk], column factors fp16 [dv]; 2 = codes
 *                   [dk, dv/4] (u = (z+3)/2), row factors fp16 [dk, dv/32], column factors fp16 [dv]
 *   qoff + h*qsz    (pw only) head h's window: P e4m3 [m, dk], V e4m3 [m, dv], PS fp32 [m], VS fp32 [m]
 * offs, bits [hv] int32 and w [hv, dk] fp32 (row impact factors of the fit) are device arrays of the layer's plan.
 * blob / slot_stride: base of slot 0 and bytes per slot (both multiples of 16). */
typedef struct sq_gga_slots {
    void* blob;         int64_t slot_stride;
    const int32_t* offs;
    const int32_t* bits;
    const float* w;
    int32_t hv, hk, dk, dv;
    int32_t m;          /* window length (pw), <= 8 */
    int32_t pw;         /* 1: the FP8 write window is kept; 0: every token's write goes into the state */
    int64_t qoff, qsz;
} sq_gga_slots;

/* One decode token per batch row on slots idx[b] (idx required; <= 0: padding).  q, k [rows, hk, dk] (normalised in
 * the kernel, q also times `scale`), v [rows, hv, dv] with row strides in elements; out [rows, hv, dv] contiguous.
 * gate = 1: a, b [rows, hv], A_log, dt_bias [hv] (decay exp(-exp(A_log) softplus(a + dt_bias)), beta = sigmoid(b));
 * gate = 0: g (log decay) and beta [rows, hv].  With pw the slots' counters are advanced by a second small launch. */
typedef struct sq_gga_args {
    sq_gga_slots sl;
    int32_t rows;
    const int32_t* idx;
    const void* q;      int64_t s_q;     int32_t q_dtype;
    const void* k;      int64_t s_k;     int32_t k_dtype;
    const void* v;      int64_t s_v;     int32_t v_dtype;
    int32_t gate;
    const void* g;      int64_t s_g;     int32_t g_dtype;
    const void* beta;   int64_t s_beta;  int32_t beta_dtype;
    const void* a;      int64_t s_a;     int32_t a_dtype;
    const void* b;      int64_t s_b;     int32_t b_dtype;
    const void* A_log;  int32_t A_log_dtype;
    const void* dt_bias; int32_t dt_bias_dtype;
    void* out;          int32_t out_dtype;
    float scale;
} sq_gga_args;

int sq_abi_version(void);
const char* sq_strerror(int code);
const char* sq_last_error(void);

/* Diagnostic, no counterpart in the reference: several compiled kernel instances can serve the same step call (one
 * with the serving dtypes compiled in or the general one; a workgroup per key head or a wavefront per head; how many
 * value heads a workgroup takes).  Results do not depend on the choice up to the accumulation order of fp32 sums; the
 * twin tests and the profiling scripts use this to compare instances.  Non-zero no_specialised / no_group_kernel
 * exclude those instances, max_heads_per_workgroup <= 0 means no cap, lds_pad_bytes > 0 adds that much unused dynamic
 * LDS to the workgroup-per-key-head launches (fewer resident workgroups per compute unit; static + dynamic must stay
 * within 64 KB or the launch fails).  Process-wide, takes effect on the next call; the library reads no environment
 * variable.  Pure host code. */
void sq_debug_select(int32_t no_specialised, int32_t no_group_kernel, int32_t max_heads_per_workgroup,
                     int32_t lds_pad_bytes);

/* 1 if a kernel is built for this layout (family: 0 GDN, 1 KDA, 2 Mamba2), else 0. Pure host code. */
int sq_supported(int family, const sq_layout* lay);

int sq_gdn_step(const sq_gdn_args* args, void* stream);
int sq_kda_step(const sq_kda_args* args, void* stream);
int sq_mamba2_step(const sq_mamba2_args* args, void* stream);
int sq_pack_vk(const sq_pack_args* args, void* stream);
/* order[0 .. rows) <- a dispatch order for the step calls' `order` (no counterpart in the reference): the rows whose
 * buffer fills on the coming step (NPTR[idx[b] * sN] & (m-1) == m-1; idx == NULL: sequence b) dealt evenly over the
 * eight ranges of rows that the step kernels give to the GPU's eight dies, and inside a range one after every few
 * other rows of its first quarter; the other rows, padding rows (idx[b] <= 0) included, in batch order.  The identity
 * when rows is not a multiple of 8 or below 64, when no row folds, or when more than every second row does.  NPTR and
 * sN (in elements) as in sq_state; one small launch.  The counters of all layers of a model move together, so one
 * list per decode step serves every layer. */
int sq_fold_order(const int32_t* idx, const int32_t* NPTR, int64_t sN, int32_t m, int32_t rows, int32_t* order,
                  void* stream);
int sq_read(const sq_read_args* args, void* stream);
int sq_gga_step(const sq_gga_args* args, void* stream);
/* Fit + pack canonical fp32 states X [rows, hv, dk, dv] (key-major, contiguous) into slots idx[b]; their counters are
 * zeroed (the window starts empty).  Rows with idx[b] <= 0 are skipped. */
int sq_gga_store(const sq_gga_slots* slots, const int32_t* idx, int32_t rows, const float* X, void* stream);
/* The stored states of slots idx[b] (without the window) as canonical fp32 Y [rows, hv, dk, dv]; zeros for
 * idx[b] <= 0. */
int sq_gga_load(const sq_gga_slots* slots, const int32_t* idx, int32_t rows, float* Y, void* stream);
/* 1 if the GGA kernels are built for these head dims and window length. Pure host code. */
int sq_gga_supported(int32_t dk, int32_t dv, int32_t m);

#ifdef __cplusplus
}
#endif
#endif /* STATEQUANT_HIP_H */
