// extern "C" surface of libsqhip.so (declared in include/statequant_hip.h): argument validation, translation of the
// public structs into kernel parameter blocks, error reporting.  No allocation, no synchronization.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "../../include/statequant_hip.h"
#include "sq_params.h"

namespace {

thread_local char g_err[256] = "";

int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

bool pow2(int n) { return n > 0 && (n & (n - 1)) == 0; }
bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
bool dtype_ok(int d) { return d == SQ_F32 || d == SQ_BF16 || d == SQ_F16; }

// Geometry / format checks shared by the three families; fills the LayoutKey part of a parameter block.
int check_layout(const sq_layout& L, const char* who, sq::LayoutKey* key) {
    if (L.bits != 4 && L.bits != 8 && L.bits != 16 && L.bits != 32)
        return fail(SQ_E_UNSUPPORTED, "%s: bits must be 4, 8 (codes), 16 (bf16 state) or 32 (fp32 state), got %d", who,
                    L.bits);
    const bool flt = L.bits >= 16;                        // unquantized state: no scales, group / axis ignored
    if (!flt && !pow2(L.group)) return fail(SQ_E_ARG, "%s: group %d is not a power of two", who, L.group);
    if (!flt && !L.axis_k && (L.dv <= 0 || L.dv % L.group))
        return fail(SQ_E_ARG, "%s: value-axis group %d does not divide d_v %d", who, L.group, L.dv);
    if (L.buffer_bits != 8 && L.buffer_bits != 16)
        return fail(SQ_E_ARG, "%s: buffer_bits must be 8 or 16, got %d", who, L.buffer_bits);
    if (!pow2(L.m) || L.m > 32) return fail(SQ_E_ARG, "%s: m must be a power of two <= 32, got %d", who, L.m);
    if (L.hv <= 0 || L.hk <= 0 || L.hv % L.hk) return fail(SQ_E_ARG, "%s: hv %d, hk %d", who, L.hv, L.hk);
    if (L.dk <= 0 || L.dv <= 0 || (L.dk & 1)) return fail(SQ_E_ARG, "%s: dk %d, dv %d", who, L.dk, L.dv);
    key->bits = L.bits;
    key->group = flt ? L.dk : L.group;
    key->qbuf = L.buffer_bits == 8;
    key->m = L.m;
    key->hv = L.hv;
    key->hk = L.hk;
    key->dk = L.dk;
    key->dv = L.dv;
    key->axv = (flt || L.axis_k) ? 0 : 1;
    key->gqa = L.hv / L.hk;
    key->hv_shift = pow2(L.hv) ? __builtin_ctz(unsigned(L.hv)) : -1;
    key->gqa_shift = pow2(key->gqa) ? __builtin_ctz(unsigned(key->gqa)) : -1;
    key->per_xcd = 0;
    return SQ_OK;
}

// Tiles per XCD for the launch's tile -> XCD mapping (0: tile count not a multiple of 8, workgroup id = tile id).
void set_rows(sq::LayoutKey* key, int rows) {
    const int64_t tiles = int64_t(rows) * key->hv;
    key->per_xcd = (tiles % 8 == 0) ? int(tiles / 8) : 0;
}

// A per-sequence or per-row stride as the kernels take it: non-negative, below 2^31.
bool stride_ok(int64_t s) { return s >= 0 && s < (int64_t(1) << 31); }

// Pointers, strides and alignment of the stored state.  The kernels read a lane's piece of a code row with one
// 128-bit (int8) or 64-bit (int4) load and a piece of a buffered int8 key with one 128-bit load.
int check_state(const sq_state& s, const sq_layout& L, const char* who, sq::StatePtrs* st) {
    const bool flt = L.bits >= 16;
    if (!s.S || (!flt && !s.SC) || !s.KB || !s.UB || !s.GB || !s.GCUR || !s.NPTR)
        return fail(SQ_E_ARG, "%s: null state pointer", who);
    if (L.buffer_bits == 8 && (!s.KBS || !s.UBS)) return fail(SQ_E_ARG, "%s: int8 buffer without scales", who);
    const size_t row_align = L.bits == 4 ? 8 : 16;
    const int64_t s_bytes = s.sS * (flt ? L.bits / 8 : 1);          // the kernels address the state in bytes
    if (!aligned(s.S, row_align) || (s_bytes % int64_t(row_align)))
        return fail(SQ_E_ARG, "%s: state must be %zu-byte aligned (base and per-sequence stride)", who, row_align);
    if (L.buffer_bits == 8 && (!aligned(s.KB, 16) || (s.sKB % 16)))
        return fail(SQ_E_ARG, "%s: int8 key buffer must be 16-byte aligned (base and per-sequence stride)", who);
    // scales and buffered values are staged into LDS with 128-bit loads
    if ((!flt && (!aligned(s.SC, 16) || (s.sSC % 8))) || !aligned(s.UB, 16) || ((s.sUB * (L.buffer_bits / 8)) % 16))
        return fail(SQ_E_ARG, "%s: scales and value buffer must be 16-byte aligned (base and per-sequence stride)",
                    who);
    if (!aligned(s.GB, 4) || !aligned(s.GCUR, 4) || !aligned(s.NPTR, 4))
        return fail(SQ_E_ARG, "%s: misaligned decay / counter pointer", who);
    if (!stride_ok(s_bytes) || !stride_ok(s.sSC) || !stride_ok(s.sKB) || !stride_ok(s.sKBS) || !stride_ok(s.sUB) ||
        !stride_ok(s.sUBS) || !stride_ok(s.sGB) || !stride_ok(s.sGC) || !stride_ok(s.sN))
        return fail(SQ_E_ARG, "%s: per-sequence strides must be in [0, 2^31)", who);
    st->S = static_cast<uint8_t*>(s.S);         st->sS = uint32_t(s_bytes);
    st->SC = static_cast<uint16_t*>(s.SC);      st->sSC = uint32_t(s.sSC);
    st->KB = static_cast<uint8_t*>(s.KB);       st->sKB = uint32_t(s.sKB);
    st->KBS = static_cast<uint16_t*>(s.KBS);    st->sKBS = uint32_t(s.sKBS);
    st->UB = static_cast<uint8_t*>(s.UB);       st->sUB = uint32_t(s.sUB);
    st->UBS = static_cast<uint16_t*>(s.UBS);    st->sUBS = uint32_t(s.sUBS);
    st->GB = s.GB;                              st->sGB = uint32_t(s.sGB);
    st->GCUR = s.GCUR;                          st->sGC = uint32_t(s.sGC);
    st->NPTR = s.NPTR;                          st->sN = uint32_t(s.sN);
    return SQ_OK;
}

int finish(int rc, const char* who, const sq_layout& L) {
    if (rc == 0) return SQ_OK;
    if (rc == -1)
        return fail(SQ_E_UNSUPPORTED, "%s: no kernel built for int%d group %d, d_k %d, d_v %d, m %d, buffer_bits %d",
                    who, L.bits, L.group, L.dk, L.dv, L.m, L.buffer_bits);
    return fail(SQ_E_LAUNCH, "%s: %s", who, hipGetErrorString(hipError_t(rc)));
}

#define SQ_TRY(expr)              \
    do {                          \
        const int rc_ = (expr);   \
        if (rc_ != SQ_OK) return rc_; \
    } while (0)

}  // namespace

extern "C" {

int sq_abi_version(void) { return SQ_ABI_VERSION; }

void sq_debug_select(int32_t no_specialised, int32_t no_group_kernel, int32_t max_heads_per_workgroup,
                     int32_t lds_pad_bytes) {
    sq::select_instances(no_specialised, no_group_kernel, max_heads_per_workgroup, lds_pad_bytes);
}

const char* sq_strerror(int code) {
    switch (code) {
        case SQ_OK: return "ok";
        case SQ_E_ARG: return "invalid argument";
        case SQ_E_UNSUPPORTED: return "unsupported layout";
        case SQ_E_LAUNCH: return "kernel launch failed";
        default: return "unknown error";
    }
}

const char* sq_last_error(void) { return g_err; }

int sq_supported(int family, const sq_layout* lay) {
    if (!lay) return 0;
    sq::LayoutKey key;
    if (check_layout(*lay, "sq_supported", &key) != SQ_OK) return 0;
    if (family == 0) {
        sq::GdnParams p{};
        static_cast<sq::LayoutKey&>(p) = key;
        return sq::dispatch_gdn(p, nullptr, false) == 0;
    }
    if (family == 1) {
        sq::KdaParams p{};
        static_cast<sq::LayoutKey&>(p) = key;
        return sq::dispatch_kda(p, nullptr, false) == 0;
    }
    if (family == 2) {
        sq::Mamba2Params p{};
        static_cast<sq::LayoutKey&>(p) = key;
        return sq::dispatch_mamba2(p, nullptr, false) == 0;
    }
    return 0;
}

int sq_gdn_step(const sq_gdn_args* a, void* stream) {
    const char* who = "sq_gdn_step";
    if (!a) return fail(SQ_E_ARG, "%s: null args", who);
    sq::GdnParams p{};
    SQ_TRY(check_layout(a->lay, who, &p));
    if (a->rows < 0) return fail(SQ_E_ARG, "%s: rows %d", who, a->rows);
    if (a->rows == 0) return SQ_OK;
    SQ_TRY(check_state(a->st, a->lay, who, &p.st));
    if (!a->q || !a->k || !a->v || !a->out) return fail(SQ_E_ARG, "%s: null q / k / v / out", who);
    if (!dtype_ok(a->q_dtype) || !dtype_ok(a->k_dtype) || !dtype_ok(a->v_dtype) || !dtype_ok(a->out_dtype))
        return fail(SQ_E_ARG, "%s: bad dtype code", who);
    if (a->gate) {
        if (!a->a || !a->b || !a->A_log || !a->dt_bias)
            return fail(SQ_E_ARG, "%s: gate without a / b / A_log / dt_bias", who);
        if (!dtype_ok(a->a_dtype) || !dtype_ok(a->b_dtype) || !dtype_ok(a->A_log_dtype) || !dtype_ok(a->dt_bias_dtype))
            return fail(SQ_E_ARG, "%s: bad gate dtype code", who);
    } else {
        if (!a->g || !a->beta) return fail(SQ_E_ARG, "%s: neither g / beta nor a gate", who);
        if (!dtype_ok(a->g_dtype) || !dtype_ok(a->beta_dtype))
            return fail(SQ_E_ARG, "%s: bad g / beta dtype code", who);
    }
    if (!stride_ok(a->s_q) || !stride_ok(a->s_k) || !stride_ok(a->s_v) ||
        !stride_ok(a->gate ? a->s_a : a->s_g) || !stride_ok(a->gate ? a->s_b : a->s_beta))
        return fail(SQ_E_ARG, "%s: row strides must be in [0, 2^31)", who);
    if (a->order && !aligned(a->order, 4)) return fail(SQ_E_ARG, "%s: misaligned order", who);
    p.rows = a->rows;
    set_rows(&p, a->rows);
    p.idx = a->idx;
    p.order = a->order;
    p.q = a->q; p.s_q = uint32_t(a->s_q); p.q_dt = a->q_dtype;
    p.k = a->k; p.s_k = uint32_t(a->s_k); p.k_dt = a->k_dtype;
    p.v = a->v; p.s_v = uint32_t(a->s_v); p.v_dt = a->v_dtype;
    p.qk_per_key_head = a->qk_per_key_head != 0;
    p.gate = a->gate != 0;
    if (p.gate) {
        p.a = a->a; p.s_a = uint32_t(a->s_a); p.a_dt = a->a_dtype;
        p.bt = a->b; p.s_bt = uint32_t(a->s_b); p.bt_dt = a->b_dtype;
        p.A_log = a->A_log; p.A_log_dt = a->A_log_dtype;
        p.dt_bias = a->dt_bias; p.dt_bias_dt = a->dt_bias_dtype;
    } else {                  // the kernel reads the same four operands either way: g, beta, and g twice as dummies
        p.a = a->g; p.s_a = uint32_t(a->s_g); p.a_dt = a->g_dtype;
        p.bt = a->beta; p.s_bt = uint32_t(a->s_beta); p.bt_dt = a->beta_dtype;
        p.A_log = a->g; p.A_log_dt = a->g_dtype;
        p.dt_bias = a->g; p.dt_bias_dt = a->g_dtype;
    }
    p.out = a->out; p.out_dt = a->out_dtype;
    p.scale = a->scale;
    return finish(sq::dispatch_gdn(p, static_cast<hipStream_t>(stream), true), who, a->lay);
}

int sq_kda_step(const sq_kda_args* a, void* stream) {
    const char* who = "sq_kda_step";
    if (!a) return fail(SQ_E_ARG, "%s: null args", who);
    sq::KdaParams p{};
    SQ_TRY(check_layout(a->lay, who, &p));
    if (a->lay.hk != a->lay.hv)
        return fail(SQ_E_ARG, "%s: KDA has no grouped keys (hk %d != hv %d)", who, a->lay.hk, a->lay.hv);
    if (a->rows < 0) return fail(SQ_E_ARG, "%s: rows %d", who, a->rows);
    if (a->rows == 0) return SQ_OK;
    SQ_TRY(check_state(a->st, a->lay, who, &p.st));
    if (!aligned(a->st.GB, 16) || (a->st.sGB % 4))
        return fail(SQ_E_ARG, "%s: GB must be 16-byte aligned (base and per-sequence stride)", who);
    if (!a->q || !a->k || !a->v || !a->g || !a->beta || !a->out) return fail(SQ_E_ARG, "%s: null input / output", who);
    if (!dtype_ok(a->q_dtype) || !dtype_ok(a->k_dtype) || !dtype_ok(a->v_dtype) || !dtype_ok(a->g_dtype) ||
        !dtype_ok(a->beta_dtype) || !dtype_ok(a->out_dtype))
        return fail(SQ_E_ARG, "%s: bad dtype code", who);
    if (!stride_ok(a->s_q) || !stride_ok(a->s_k) || !stride_ok(a->s_v) || !stride_ok(a->s_g) ||
        !stride_ok(a->s_beta) || !stride_ok(a->s_out))
        return fail(SQ_E_ARG, "%s: row strides must be in [0, 2^31)", who);
    if (a->order && !aligned(a->order, 4)) return fail(SQ_E_ARG, "%s: misaligned order", who);
    p.rows = a->rows;
    set_rows(&p, a->rows);
    p.idx = a->idx;
    p.order = a->order;
    p.q = a->q; p.s_q = uint32_t(a->s_q); p.q_dt = a->q_dtype;
    p.k = a->k; p.s_k = uint32_t(a->s_k); p.k_dt = a->k_dtype;
    p.v = a->v; p.s_v = uint32_t(a->s_v); p.v_dt = a->v_dtype;
    p.g = a->g; p.s_g = uint32_t(a->s_g); p.g_dt = a->g_dtype;
    p.beta = a->beta; p.s_beta = uint32_t(a->s_beta); p.beta_dt = a->beta_dtype;
    p.out = a->out; p.s_out = uint32_t(a->s_out); p.out_dt = a->out_dtype;
    p.scale = a->scale;
    return finish(sq::dispatch_kda(p, static_cast<hipStream_t>(stream), true), who, a->lay);
}

int sq_mamba2_step(const sq_mamba2_args* a, void* stream) {
    const char* who = "sq_mamba2_step";
    if (!a) return fail(SQ_E_ARG, "%s: null args", who);
    sq::Mamba2Params p{};
    SQ_TRY(check_layout(a->lay, who, &p));
    if (a->rows < 0) return fail(SQ_E_ARG, "%s: rows %d", who, a->rows);
    if (a->rows == 0) return SQ_OK;
    SQ_TRY(check_state(a->st, a->lay, who, &p.st));
    if (!a->x || !a->dt || !a->B || !a->C || !a->A || !a->out) return fail(SQ_E_ARG, "%s: null input / output", who);
    if (!dtype_ok(a->x_dtype) || !dtype_ok(a->dt_dtype) || !dtype_ok(a->B_dtype) || !dtype_ok(a->C_dtype) ||
        !dtype_ok(a->A_dtype) || !dtype_ok(a->out_dtype) || (a->D && !dtype_ok(a->D_dtype)) ||
        (a->dt_bias && !dtype_ok(a->dt_bias_dtype)))
        return fail(SQ_E_ARG, "%s: bad dtype code", who);
    if (!stride_ok(a->s_x) || !stride_ok(a->s_dt) || !stride_ok(a->s_B) || !stride_ok(a->s_C) || !stride_ok(a->s_out))
        return fail(SQ_E_ARG, "%s: row strides must be in [0, 2^31)", who);
    if (a->order && !aligned(a->order, 4)) return fail(SQ_E_ARG, "%s: misaligned order", who);
    p.rows = a->rows;
    set_rows(&p, a->rows);
    p.idx = a->idx;
    p.order = a->order;
    p.x = a->x; p.s_x = uint32_t(a->s_x); p.x_dt = a->x_dtype;
    p.dt = a->dt; p.s_dt = uint32_t(a->s_dt); p.dt_dt = a->dt_dtype;
    p.B = a->B; p.s_B = uint32_t(a->s_B); p.B_dt = a->B_dtype;
    p.C = a->C; p.s_C = uint32_t(a->s_C); p.C_dt = a->C_dtype;
    p.A = a->A; p.A_dt = a->A_dtype;
    p.has_D = a->D != nullptr;
    p.has_dt_bias = a->dt_bias != nullptr;
    p.D = p.has_D ? a->D : a->A;
    p.D_dt = p.has_D ? a->D_dtype : a->A_dtype;
    p.dt_bias = p.has_dt_bias ? a->dt_bias : a->A;
    p.dt_bias_dt = p.has_dt_bias ? a->dt_bias_dtype : a->A_dtype;
    p.dt_softplus = a->dt_softplus != 0;
    p.dt_clamp = a->dt_clamp != 0;
    p.dt_min = a->dt_min; p.dt_max = a->dt_max;
    p.out = a->out; p.s_out = uint32_t(a->s_out); p.out_dt = a->out_dtype;
    return finish(sq::dispatch_mamba2(p, static_cast<hipStream_t>(stream), true), who, a->lay);
}

int sq_pack_vk(const sq_pack_args* a, void* stream) {
    const char* who = "sq_pack_vk";
    if (!a) return fail(SQ_E_ARG, "%s: null args", who);
    const sq_layout& L = a->lay;
    if (L.bits != 4 && L.bits != 8 && L.bits != 16 && L.bits != 32)
        return fail(SQ_E_UNSUPPORTED, "%s: bits must be 4, 8, 16 or 32, got %d", who, L.bits);
    const bool flt = L.bits >= 16;
    if (L.hv <= 0 || L.dk <= 0 || L.dv <= 0) return fail(SQ_E_ARG, "%s: hv %d, dk %d, dv %d", who, L.hv, L.dk, L.dv);
    if (!flt && !L.axis_k && (L.group <= 0 || L.dv % L.group))
        return fail(SQ_E_ARG, "%s: value-axis group %d does not divide d_v %d", who, L.group, L.dv);
    if (a->rows < 0) return fail(SQ_E_ARG, "%s: rows %d", who, a->rows);
    if (a->rows == 0) return SQ_OK;
    if (!a->src || !a->S || (!flt && !a->SC)) return fail(SQ_E_ARG, "%s: null src / S / SC", who);
    const size_t row_align = L.bits == 4 ? 8 : 16;
    const int64_t s_bytes = a->sS * (flt ? L.bits / 8 : 1);          // the kernels address the state in bytes
    if (!aligned(a->src, 16) || (a->s_src % 4) || !aligned(a->S, row_align) || (s_bytes % int64_t(row_align)) ||
        (!flt && (!aligned(a->SC, 4) || (a->sSC % 2))))
        return fail(SQ_E_ARG, "%s: src must be 16-byte aligned, the state %zu-byte, scales 4-byte aligned", who,
                    row_align);
    if (!stride_ok(a->s_src) || !stride_ok(s_bytes) || !stride_ok(a->sSC) || !stride_ok(a->sGC) || !stride_ok(a->sN))
        return fail(SQ_E_ARG, "%s: strides must be in [0, 2^31)", who);
    if (a->GCUR && a->gcur_per_head <= 0) return fail(SQ_E_ARG, "%s: gcur_per_head %d", who, a->gcur_per_head);
    sq::PackParams p{};
    p.bits = L.bits; p.group = flt ? L.dk : L.group; p.axv = (flt || L.axis_k) ? 0 : 1;
    p.hv = L.hv; p.dk = L.dk; p.dv = L.dv;
    p.rows = a->rows; p.idx = a->idx;
    p.src = a->src; p.s_src = uint32_t(a->s_src);
    p.S = static_cast<uint8_t*>(a->S); p.sS = uint32_t(s_bytes);
    p.SC = static_cast<uint16_t*>(a->SC); p.sSC = uint32_t(a->sSC);
    p.GCUR = a->GCUR; p.sGC = uint32_t(a->sGC); p.gcur_per_head = a->gcur_per_head;
    p.NPTR = a->NPTR; p.sN = uint32_t(a->sN);
    p.nptr_copies = a->nptr_copies > a->lay.hv ? a->nptr_copies : a->lay.hv;
    if (a->NPTR && a->sN != 0 && int64_t(p.nptr_copies) > a->sN)
        return fail(SQ_E_ARG, "%s: %d counter copies do not fit a counter stride of %lld", who, p.nptr_copies, (long long)a->sN);
    return finish(sq::dispatch_pack(p, static_cast<hipStream_t>(stream), true), who, a->lay);
}

int sq_fold_order(const int32_t* idx, const int32_t* NPTR, int64_t sN, int32_t m, int32_t rows, int32_t* order,
                  void* stream) {
    const char* who = "sq_fold_order";
    if (rows < 0) return fail(SQ_E_ARG, "%s: rows %d", who, rows);
    if (rows == 0) return SQ_OK;
    if (!NPTR || !order || !aligned(NPTR, 4) || !aligned(order, 4) || (idx && !aligned(idx, 4)))
        return fail(SQ_E_ARG, "%s: null or misaligned NPTR / order / idx", who);
    if (m < 1 || (m & (m - 1))) return fail(SQ_E_ARG, "%s: m %d is not a power of two", who, m);
    if (!stride_ok(sN)) return fail(SQ_E_ARG, "%s: counter stride must be in [0, 2^31)", who);
    const int rc = sq::launch_fold_order(idx, NPTR, uint32_t(sN), m, rows, order, static_cast<hipStream_t>(stream));
    if (rc != 0) return fail(SQ_E_LAUNCH, "%s: %s", who, hipGetErrorString(hipError_t(rc)));
    return SQ_OK;
}

int sq_read(const sq_read_args* a, void* stream) {
    const char* who = "sq_read";
    if (!a) return fail(SQ_E_ARG, "%s: null args", who);
    sq::ReadParams p{};
    SQ_TRY(check_layout(a->lay, who, &p));
    if (a->lay.m > 16) return fail(SQ_E_UNSUPPORTED, "%s: m %d > 16", who, a->lay.m);
    if (a->kda && a->lay.hk != a->lay.hv) return fail(SQ_E_ARG, "%s: KDA has no grouped keys", who);
    if (a->rows < 0) return fail(SQ_E_ARG, "%s: rows %d", who, a->rows);
    if (a->rows == 0) return SQ_OK;
    SQ_TRY(check_state(a->st, a->lay, who, &p.st));
    if (a->kda && (!aligned(a->st.GB, 4) || !aligned(a->st.GCUR, 4)))
        return fail(SQ_E_ARG, "%s: misaligned decay", who);
    if (!a->out || !aligned(a->out, 16) || (a->s_out % 4) || !stride_ok(a->s_out))
        return fail(SQ_E_ARG, "%s: out must be 16-byte aligned with a row stride in [0, 2^31)", who);
    p.kda = a->kda != 0;
    p.rows = a->rows; p.idx = a->idx;
    p.out = a->out; p.s_out = uint32_t(a->s_out);
    return finish(sq::dispatch_read(p, static_cast<hipStream_t>(stream), true), who, a->lay);
}

namespace {
int check_gga_slots(const sq_gga_slots& s, const char* who, sq::GgaParams* p) {
    if (!s.blob || !s.offs || !s.bits || !s.w) return fail(SQ_E_ARG, "%s: null blob / offs / bits / w", who);
    if (!aligned(s.blob, 16) || s.slot_stride <= 0 || (s.slot_stride % 16))
        return fail(SQ_E_ARG, "%s: blob and slot stride must be multiples of 16 bytes", who);
    if (s.hv <= 0 || s.hk <= 0 || s.hv % s.hk) return fail(SQ_E_ARG, "%s: hv %d, hk %d", who, s.hv, s.hk);
    if (s.pw && (s.m < 1 || s.qoff <= 0 || (s.qoff % 16) || s.qsz < int64_t(s.m) * (s.dk + s.dv + 8) ||
                 s.qoff + int64_t(s.hv) * s.qsz > s.slot_stride || s.qoff >= (int64_t(1) << 31) ||
                 s.qsz >= (int64_t(1) << 31)))
        return fail(SQ_E_ARG, "%s: window of m %d at qoff %lld, qsz %lld does not fit the slot", who, s.m,
                    (long long)s.qoff, (long long)s.qsz);
    p->blob = static_cast<uint8_t*>(s.blob);
    p->slot_stride = uint64_t(s.slot_stride);
    p->offs = s.offs;
    p->bits = s.bits;
    p->w = s.w;
    p->hv = s.hv; p->hk = s.hk; p->gqa = s.hv / s.hk; p->dk = s.dk; p->dv = s.dv;
    p->pw = s.pw != 0;
    p->m = p->pw ? s.m : 1;
    p->qoff = uint32_t(s.pw ? s.qoff : 0);
    p->qsz = uint32_t(s.pw ? s.qsz : 0);
    if (sq::dispatch_gga(*p, 0, nullptr, false) != 0)
        return fail(SQ_E_UNSUPPORTED, "%s: no kernel built for d_k %d, d_v %d, window %d", who, s.dk, s.dv, p->m);
    return SQ_OK;
}
int finish_gga(int rc, const char* who) {
    if (rc == 0) return SQ_OK;
    return fail(SQ_E_LAUNCH, "%s: %s", who, hipGetErrorString(hipError_t(rc)));
}
}  // namespace

int sq_gga_supported(int32_t dk, int32_t dv, int32_t m) {
    sq::GgaParams p{};
    p.dk = dk; p.dv = dv; p.m = m;
    return sq::dispatch_gga(p, 0, nullptr, false) == 0;
}

int sq_gga_step(const sq_gga_args* a, void* stream) {
    const char* who = "sq_gga_step";
    if (!a) return fail(SQ_E_ARG, "%s: null args", who);
    if (a->rows < 0) return fail(SQ_E_ARG, "%s: rows %d", who, a->rows);
    if (a->rows == 0) return SQ_OK;
    sq::GgaParams p{};
    SQ_TRY(check_gga_slots(a->sl, who, &p));
    if (!a->idx || !a->q || !a->k || !a->v || !a->out) return fail(SQ_E_ARG, "%s: null idx / q / k / v / out", who);
    if (!dtype_ok(a->q_dtype) || !dtype_ok(a->k_dtype) || !dtype_ok(a->v_dtype) || !dtype_ok(a->out_dtype))
        return fail(SQ_E_ARG, "%s: bad dtype code", who);
    if (a->gate) {
        if (!a->a || !a->b || !a->A_log || !a->dt_bias)
            return fail(SQ_E_ARG, "%s: gate without a / b / A_log / dt_bias", who);
        if (!dtype_ok(a->a_dtype) || !dtype_ok(a->b_dtype) || !dtype_ok(a->A_log_dtype) || !dtype_ok(a->dt_bias_dtype))
            return fail(SQ_E_ARG, "%s: bad gate dtype code", who);
    } else {
        if (!a->g || !a->beta) return fail(SQ_E_ARG, "%s: neither g / beta nor a gate", who);
        if (!dtype_ok(a->g_dtype) || !dtype_ok(a->beta_dtype))
            return fail(SQ_E_ARG, "%s: bad g / beta dtype code", who);
    }
    if (!stride_ok(a->s_q) || !stride_ok(a->s_k) || !stride_ok(a->s_v) ||
        !stride_ok(a->gate ? a->s_a : a->s_g) || !stride_ok(a->gate ? a->s_b : a->s_beta))
        return fail(SQ_E_ARG, "%s: row strides must be in [0, 2^31)", who);
    p.rows = a->rows;
    p.idx = a->idx;
    p.q = a->q; p.s_q = uint32_t(a->s_q); p.q_dt = a->q_dtype;
    p.k = a->k; p.s_k = uint32_t(a->s_k); p.k_dt = a->k_dtype;
    p.v = a->v; p.s_v = uint32_t(a->s_v); p.v_dt = a->v_dtype;
    p.gate = a->gate != 0;
    if (p.gate) {
        p.a = a->a; p.s_a = uint32_t(a->s_a); p.a_dt = a->a_dtype;
        p.bt = a->b; p.s_bt = uint32_t(a->s_b); p.bt_dt = a->b_dtype;
        p.A_log = a->A_log; p.A_log_dt = a->A_log_dtype;
        p.dt_bias = a->dt_bias; p.dt_bias_dt = a->dt_bias_dtype;
    } else {
        p.a = a->g; p.s_a = uint32_t(a->s_g); p.a_dt = a->g_dtype;
        p.bt = a->beta; p.s_bt = uint32_t(a->s_beta); p.bt_dt = a->beta_dtype;
        p.A_log = a->g; p.A_log_dt = a->g_dtype;
        p.dt_bias = a->g; p.dt_bias_dt = a->g_dtype;
    }
    p.out = a->out; p.out_dt = a->out_dtype;
    p.scale = a->scale;
    return finish_gga(sq::dispatch_gga(p, 0, static_cast<hipStream_t>(stream), true), who);
}

int sq_gga_store(const sq_gga_slots* s, const int32_t* idx, int32_t rows, const float* X, void* stream) {
    const char* who = "sq_gga_store";
    if (!s) return fail(SQ_E_ARG, "%s: null slots", who);
    if (rows < 0) return fail(SQ_E_ARG, "%s: rows %d", who, rows);
    if (rows == 0) return SQ_OK;
    sq::GgaParams p{};
    SQ_TRY(check_gga_slots(*s, who, &p));
    if (!idx || !X || !aligned(X, 16)) return fail(SQ_E_ARG, "%s: null idx / X, or X not 16-byte aligned", who);
    p.rows = rows;
    p.idx = idx;
    p.X = X;
    return finish_gga(sq::dispatch_gga(p, 1, static_cast<hipStream_t>(stream), true), who);
}

int sq_gga_load(const sq_gga_slots* s, const int32_t* idx, int32_t rows, float* Y, void* stream) {
    const char* who = "sq_gga_load";
    if (!s) return fail(SQ_E_ARG, "%s: null slots", who);
    if (rows < 0) return fail(SQ_E_ARG, "%s: rows %d", who, rows);
    if (rows == 0) return SQ_OK;
    sq::GgaParams p{};
    SQ_TRY(check_gga_slots(*s, who, &p));
    if (!idx || !Y || !aligned(Y, 16)) return fail(SQ_E_ARG, "%s: null idx / Y, or Y not 16-byte aligned", who);
    p.rows = rows;
    p.idx = idx;
    p.Y = Y;
    return finish_gga(sq::dispatch_gga(p, 2, static_cast<hipStream_t>(stream), true), who);
}

}  // extern "C"
