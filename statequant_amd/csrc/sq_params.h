// Kernel-side argument blocks (typed, validated copies of the public structs in include/statequant_hip.h) and the
// per-family dispatchers that map a layout onto a compiled kernel instance.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sq {

// Per-sequence strides are below 2^31 (checked by the C ABI): sequence x stride is then one 32 x 32 -> 64 bit
// multiply on the scalar unit instead of a full 64-bit one.
struct StatePtrs {
    uint8_t* S;      uint32_t sS;     // bytes of codes per sequence (int8: elements = bytes; int4: packed bytes)
    uint16_t* SC;    uint32_t sSC;
    uint8_t* KB;     uint32_t sKB;    // strides of KB / UB in ELEMENTS (int8 or bf16)
    uint16_t* KBS;   uint32_t sKBS;
    uint8_t* UB;     uint32_t sUB;
    uint16_t* UBS;   uint32_t sUBS;
    float* GB;       uint32_t sGB;
    float* GCUR;     uint32_t sGC;
    int32_t* NPTR;   uint32_t sN;
};

struct LayoutKey {
    int bits, group, qbuf, m, hv, hk, dk, dv;
    int axv;                                      // scale groups along the value axis (else along d_k)
    // launch geometry helpers, filled by the C ABI: gqa = hv / hk; log2 of hv and of gqa where they are powers of
    // two (else -1: the kernel divides), and tiles per XCD when the tile count is a multiple of 8 (else 0: no XCD
    // mapping)
    int gqa, hv_shift, gqa_shift, per_xcd;
};

struct GdnParams : LayoutKey {
    StatePtrs st;
    int rows;
    const int32_t* idx;
    const int32_t* order;                         // optional: the batch row of each position of the launch (null: natural)
    const void *q, *k, *v;
    uint32_t s_q, s_k, s_v;
    int q_dt, k_dt, v_dt;
    int qk_per_key_head, gate;
    // gate: a, b, A_log, dt_bias;  no gate: a = g, bt = beta, A_log = dt_bias = g (never used, always readable)
    const void *a, *bt, *A_log, *dt_bias;
    uint32_t s_a, s_bt;
    int a_dt, bt_dt, A_log_dt, dt_bias_dt;
    void* out;
    int out_dt;
    float scale;
};

struct KdaParams : LayoutKey {
    StatePtrs st;
    int rows;
    const int32_t* idx;
    const int32_t* order;
    const void *q, *k, *v, *g, *beta;
    uint32_t s_q, s_k, s_v, s_g, s_beta;
    int q_dt, k_dt, v_dt, g_dt, beta_dt;
    void* out;
    uint32_t s_out;
    int out_dt;
    float scale;
};

struct Mamba2Params : LayoutKey {
    StatePtrs st;
    int rows;
    const int32_t* idx;
    const int32_t* order;
    const void *x, *dt, *B, *C, *A, *D, *dt_bias;
    uint32_t s_x, s_dt, s_B, s_C;
    int x_dt, dt_dt, B_dt, C_dt, A_dt, D_dt, dt_bias_dt;
    int dt_softplus, dt_clamp, has_D, has_dt_bias;      // absent D / dt_bias: pointers alias A (readable, unused)
    float dt_min, dt_max;
    void* out;
    uint32_t s_out;
    int out_dt;
};

struct PackParams {
    int bits, group, axv, hv, dk, dv;              // axv: value-axis scale groups; bits 16 / 32: unquantized state
    int rows;
    const int32_t* idx;
    const float* src;  uint32_t s_src;            // [rows, hv, dv, dk] fp32, row stride in elements
    uint8_t* S;        uint32_t sS;
    uint16_t* SC;      uint32_t sSC;
    float* GCUR;       uint32_t sGC;  int gcur_per_head;      // optional (null: leave)
    int32_t* NPTR;     uint32_t sN;   int nptr_copies;        // counter copies per sequence (>= hv)
};

struct ReadParams : LayoutKey {
    StatePtrs st;
    int kda;                                      // decays per key channel (GB [hv, m, dk], GCUR [hv, dk])
    int rows;
    const int32_t* idx;
    float* out;        uint32_t s_out;            // [rows, hv, dv, dk] fp32, row stride in elements
};

// The mixed-width GGA / STEP slot (sq_gga.cuh): one blob per slot, per-layer tables on the device.
struct GgaParams {
    uint8_t* blob;
    uint64_t slot_stride;                         // bytes
    const int32_t* idx;
    int rows;
    const int32_t* offs;                          // [hv] byte offset of each head in the slot
    const int32_t* bits;                          // [hv] width of each head: 2, 4, 6, 8 or 16 (fp16 pivot)
    const float* w;                               // [hv, dk] row impact factors of the fit
    int hv, hk, gqa, dk, dv, m, pw;
    uint32_t qoff, qsz;                           // windows: at qoff + h * qsz
    const void *q, *k, *v;
    uint32_t s_q, s_k, s_v;
    int q_dt, k_dt, v_dt;
    int gate;                                     // as in GdnParams
    const void *a, *bt, *A_log, *dt_bias;
    uint32_t s_a, s_bt;
    int a_dt, bt_dt, A_log_dt, dt_bias_dt;
    void* out;
    int out_dt;
    float scale;
    const float* X;                               // store: canonical states [rows, hv, dk, dv]
    float* Y;                                     // load
};

// The serving cases a step kernel can be compiled for (template argument SPEC; 0 = read every choice from the
// arguments): bf16 operands and output, head counts that are powers of two, and per family
//   GDN     1: g and beta given as fp32;  2: the gate formed in the kernel from bf16 a, b and fp32 A_log, dt_bias
//   KDA     1: fp32 g and beta
//   Mamba2  1: fp32 dt, A, D, dt_bias
// `serving_case` tells which one a call is (host); `assume_serving_case<SPEC>` overwrites those fields of a kernel's
// private copy of its arguments with the constants (device), after which the compiler drops the scalar branches on
// them -- about a microsecond per launch on the 128 x 128 steps.  Dtype codes: 0 fp32, 1 bf16.
inline int serving_case(const GdnParams& p) {
    if (p.hv_shift < 0 || p.gqa_shift < 0) return 0;
    if (p.q_dt != 1 || p.k_dt != 1 || p.v_dt != 1 || p.out_dt != 1) return 0;
    if (!p.gate) return (p.a_dt == 0 && p.bt_dt == 0) ? 1 : 0;
    return (p.a_dt == 1 && p.bt_dt == 1 && p.A_log_dt == 0 && p.dt_bias_dt == 0) ? 2 : 0;
}
inline int serving_case(const KdaParams& p) {
    if (p.hv_shift < 0) return 0;
    if (p.q_dt != 1 || p.k_dt != 1 || p.v_dt != 1 || p.out_dt != 1) return 0;
    return (p.g_dt == 0 && p.beta_dt == 0) ? 1 : 0;
}
inline int serving_case(const Mamba2Params& p) {
    if (p.hv_shift < 0 || p.gqa_shift < 0) return 0;
    if (p.x_dt != 1 || p.B_dt != 1 || p.C_dt != 1 || p.out_dt != 1) return 0;
    return (p.dt_dt == 0 && p.A_dt == 0 && p.D_dt == 0 && p.dt_bias_dt == 0) ? 1 : 0;
}
template <int SPEC>
__device__ __forceinline__ void assume_serving_case(GdnParams& p) {
    if constexpr (SPEC > 0) {
        p.q_dt = p.k_dt = p.v_dt = p.out_dt = 1;
        p.a_dt = p.bt_dt = SPEC == 1 ? 0 : 1;
        p.A_log_dt = p.dt_bias_dt = 0;
        p.gate = SPEC == 2;
        __builtin_assume(p.hv_shift >= 0);
        __builtin_assume(p.gqa_shift >= 0);
    }
}
template <int SPEC>
__device__ __forceinline__ void assume_serving_case(KdaParams& p) {
    if constexpr (SPEC > 0) {
        p.q_dt = p.k_dt = p.v_dt = p.out_dt = 1;
        p.g_dt = p.beta_dt = 0;
        __builtin_assume(p.hv_shift >= 0);
    }
}
template <int SPEC>
__device__ __forceinline__ void assume_serving_case(Mamba2Params& p) {
    if constexpr (SPEC > 0) {
        p.x_dt = p.B_dt = p.C_dt = p.out_dt = 1;
        p.dt_dt = p.A_dt = p.D_dt = p.dt_bias_dt = 0;
        __builtin_assume(p.hv_shift >= 0);
        __builtin_assume(p.gqa_shift >= 0);
    }
}

// hipError_t of the launch (0 = enqueued), or -1 if no kernel is compiled for the layout.  run = false: probe only.
int dispatch_gdn(const GdnParams& p, hipStream_t stream, bool run);
int dispatch_kda(const KdaParams& p, hipStream_t stream, bool run);
int dispatch_mamba2(const Mamba2Params& p, hipStream_t stream, bool run);
int dispatch_pack(const PackParams& p, hipStream_t stream, bool run);
int dispatch_read(const ReadParams& p, hipStream_t stream, bool run);
int launch_fold_order(const int32_t* idx, const int32_t* NPTR, uint32_t sN, int m, int rows, int32_t* order,
                      hipStream_t stream);
int dispatch_gga(const GgaParams& p, int op, hipStream_t stream, bool run);      // op: 0 step, 1 store, 2 load
// Diagnostic choice among the instances that can serve a step call (behind sq_debug_select of the C ABI).
void select_instances(int no_spec, int no_quad, int ghmax, int lds_pad);
int quad_lds_pad();                                       // unused dynamic LDS added to the workgroup kernels' launches

}  // namespace sq
