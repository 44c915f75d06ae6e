// Host side of the C ABI declared in include/jlmi.h.
//
// One context = one device, one stream, one gfx950 code object loaded with
// hipModuleLoad and its kernels resolved by name.  Entry points validate
// shapes on the host before any launch (a kernel is never started on operands
// it does not fit), translate the reference's operator contracts into kernel
// launches, and report served / declined / error.  There is no CPU compute path
// here: when the code object or the device is missing, creation fails.
#include "../../include/jlmi.h"

#include <dlfcn.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <atomic>
#include <mutex>
#include <thread>
#include <string>
#include <vector>

#include "hip_api.h"
#include "kernels/args.h"
#include "scratch.h"

namespace {

thread_local std::string g_create_error;
const HipApi* H = nullptr;  // the process-wide HIP runtime, resolved by the first jl_ctx_create

struct Tuning {
    int rpw = 0, block = 0, grid = 0;
    int act_split = 0;          // grouped matvec with a gated activation: 1 always quantize it in its own launch, 2 never
    int xpre = 0;               // decode matvec: 1 / 4 float4 groups of x a thread loads ahead of its weights
    int q8pair = 0;             // Q8_0 rows: 2 keeps one block a lane-slot (2-byte-aligned loads)
    int packed_rw = 0, packed_block = 0, moe_group = 0, moe_logits = 0, moe_q6k_cols = 0;
    int moe_shares = 0;
    int gemm_rows = 0;
    int gemm_form = 0;
    int gemm_split = 0;
    int gemm_prep = 0;
    int gemm_planes = 0;
    int moe_form = 0;
    int moe_g16 = 0;
    int gemm_fold = 0, gemm_fold_waves = 0;
    int moe_chunk = 0;
    int moe_waves = 0;
    int moe_lpr = 0;
    int mx_rows = 0;
    int mx_scaled = 0;          // 1: packed MXFP4 matmul on the block-scaled fp8 x fp4 matrix instruction (lossy)
    int mx_planes = 0;          // packed MXFP4: 2 restores rows first, 3 the plane GEMM whatever the grid; 64 / 32 / 16
                                // rows a workgroup of the plane matvec
    int mx_split = 0;
};

struct Resident {
    void* dev = nullptr;
    size_t bytes = 0;
};

// A block whose feed-forward weights jl_prep_layer made resident: one device allocation, the
// pieces' addresses in it.
struct Layer {
    jl_layer_plan plan;          // host pointers cleared
    void* mem = nullptr;         // the allocation
    // packed = 0: the matrices' (banks') bytes; packed = 1: plane sets
    const void *gate = nullptr, *up = nullptr, *down = nullptr;
    const uint32_t *gp[3] = {nullptr, nullptr, nullptr}, *upl[3] = {nullptr, nullptr, nullptr},
                   *dp[3] = {nullptr, nullptr, nullptr};
    const float* norm_w = nullptr;
    const float* router = nullptr;
};

}  // namespace

struct jl_ctx {
    int device = 0;
    int act_window = 32;
    hipStream_t stream = nullptr;
    hipModule_t module = nullptr;
    std::map<std::string, hipFunction_t> fn;
    std::string err;
    std::mutex mu;  // serialises the host-pointer seam (one staging area per context)
    std::atomic<std::thread::id> mu_owner{};   // the thread inside mu (jl_forget must not try it again)
    // jl_forget only queues its range here, under a lock no launch or upload path holds; the
    // host-pointer calls apply the queue (unlink + hipFree) before their residency lookup
    std::mutex forget_mu;
    std::vector<std::pair<uintptr_t, uintptr_t>> pending_forget;
    // Q4_K matrices (device address -> rows, k) whose scales jl_fold_admit_dev found inside the
    // f16 range: the only ones the folded-scale GEMM form is used for (under forget_mu)
    std::map<uintptr_t, std::pair<int, int>> fold_ok;
    bool no_device = false;   // created with device < 0: host-side bookkeeping only
    // the static device array of scratch.hip on this context's device (null: the lookup
    // failed and static_err says why), and the state of a call that lives on it
    void* static_scratch = nullptr;
    size_t static_scratch_bytes = 0;
    std::string static_err;
    Tuning tune;
    int gemm_min_tok = 3;  // below this a per-token matvec loop is as fast (3.8 us a token against 8.9 us for up to 16)
    int num_cu = 0;
    size_t lds_limit = 0;
    std::atomic<unsigned long long> launches{0};   // kernels launched so far (jl_launch_count)

    // prefill GEMM workspace (quantized activations in stage layout), grown on demand
    void* gemm_ws = nullptr;
    size_t gemm_ws_bytes = 0;
    void* w16_ws = nullptr;   // expanded weights of the two-pass GEMM
    size_t w16_ws_bytes = 0;

    void* mx_ws = nullptr;      // partial sums of a K-split matmul (MXFP4, Q4_K)
    size_t mx_ws_bytes = 0;
    uint32_t* one_group = nullptr;   // (0, n) for n = 0..16: column ranges of a single group of n columns
    void* moe_q_ws = nullptr;   // quantized column activations of a mixture pass
    size_t moe_q_ws_bytes = 0;
    void* act_ws = nullptr;     // a long gated activation, quantized once for a grouped matvec
    size_t act_ws_bytes = 0;

    // rows restored to GGUF order for the GEMM over packed planes
    void* unpack_ws = nullptr;
    size_t unpack_ws_bytes = 0;
    void* flag_ws = nullptr;    // one word the MXFP4 packer raises when it must refuse
    size_t flag_ws_bytes = 0;

    // mixture-of-experts workspace (grouping tables and intermediate columns)
    void* moe_ws = nullptr;
    size_t moe_ws_bytes = 0;

    // blocks prepared by jl_prep_layer, and the workspace their runs share (router logits,
    // selection and weights of a mixture; gate and up of a dense block at one row)
    std::map<int, Layer> layers;
    void* layer_ws = nullptr;
    size_t layer_ws_bytes = 0;
    // a block's router logits and, when it is not handed a place for them, selection and weights
    void* moe_route_ws = nullptr;
    size_t moe_route_ws_bytes = 0;

    // host-pointer seam state
    std::map<const void*, Resident> resident;
    void* stage_x = nullptr;    // device
    void* stage_out = nullptr;  // device
    size_t stage_x_bytes = 0, stage_out_bytes = 0;
};

namespace {

// What a call in progress on THIS thread has switched on for its context: jl_reserve_shape
// walks a launch path with launching off (dry_run), jl_matmul_static_dev carves workspaces
// from the static array instead of the heap (no_alloc).  Kept per thread and tagged with the
// context, so a launch that another thread makes on the same context meanwhile is a launch.
struct CallState {
    const jl_ctx* ctx = nullptr;
    bool dry_run = false;
    bool no_alloc = false;
    size_t static_used = 0;
};
thread_local CallState g_call;
bool call_dry_run(const jl_ctx* c) { return g_call.ctx == c && g_call.dry_run; }
bool call_no_alloc(const jl_ctx* c) { return g_call.ctx == c && g_call.no_alloc; }
// Switches the state on for a scope; nests (a dry run inside a no-alloc call).
struct CallScope {
    CallState saved;
    CallScope(const jl_ctx* c, bool dry_run, bool no_alloc) : saved(g_call) {
        if (g_call.ctx != c) g_call = CallState{};
        g_call.ctx = c;
        g_call.dry_run = g_call.dry_run || dry_run;
        g_call.no_alloc = g_call.no_alloc || no_alloc;
    }
    ~CallScope() { g_call = saved; }
};

// c->mu with its owner recorded.
struct CtxLock {
    jl_ctx* c;
    explicit CtxLock(jl_ctx* ctx) : c(ctx) {
        c->mu.lock();
        c->mu_owner.store(std::this_thread::get_id());
    }
    ~CtxLock() {
        c->mu_owner.store(std::thread::id());
        c->mu.unlock();
    }
};

int fail(jl_ctx* c, int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (c) c->err = buf;
    else g_create_error = buf;
    return code;
}

#define HIP_TRY(c, call)                                                              \
    do {                                                                              \
        hipError_t e_ = (call);                                                       \
        if (e_ != hipSuccess)                                                         \
            return fail((c), JL_ERR_HIP, "%s: %s", #call, H->GetErrorString(e_));     \
    } while (0)

std::string default_code_object() {
    Dl_info info;
    if (dladdr((void*)&jl_ctx_create, &info) && info.dli_fname) {
        std::string p = info.dli_fname;
        size_t s = p.rfind('/');
        return (s == std::string::npos ? std::string(".") : p.substr(0, s)) + "/jlmi_gfx950.hsaco";
    }
    return "jlmi_gfx950.hsaco";
}

struct TypeInfo {
    const char* tag;   // kernel-name fragment
    int block_elems, block_bytes;
    int slot_elems;    // elements one lane-slot of the matvec kernel covers
};

const TypeInfo* type_info(int type) {
    static const TypeInfo q8 = {"q8_0", 32, 34, 32};
    static const TypeInfo q4k = {"q4k", 256, 144, 64};
    static const TypeInfo q6k = {"q6k", 256, 210, 64};
    switch (type) {
    case JL_TYPE_Q8_0: return &q8;
    case JL_TYPE_Q4_K: return &q4k;
    case JL_TYPE_Q6_K: return &q6k;
    }
    return nullptr;
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// Largest workgroup of the matvec variant with `rpw` rows per wavefront, 0 when the
// code object has no such variant (kernels/jlmi_kernels.hip).
int matvec_max_block(int type, int rpw, bool q8_pair = false) {
    if (rpw == 1) return 1024;
    if (rpw == 2) return type == JL_TYPE_Q6_K ? 512 : 1024;
    if (rpw == 4) return type == JL_TYPE_Q8_0 && !q8_pair ? 1024 : 512;
    return 0;
}

hipStream_t pick_stream(jl_ctx* c, void* s) { return s ? (hipStream_t)s : c->stream; }

// LDS of the decode matvec: int8 activations, a scale per 32, a sum per 16
size_t act_lds_bytes(int k) { return (size_t)k + (size_t)(k / 32) * 4 + (size_t)(k / 16) * 4; }

// Q8_0 rows in the form that takes two blocks a lane-slot with every load 4-byte aligned
// (kernels/matvec.h): rows on 4-byte boundaries, an even number of blocks a row, room in
// LDS for the second copy of the activations.
bool q8_pair_form(const jl_ctx* c, int type, const void* w, int k) {
    return type == JL_TYPE_Q8_0 && c->tune.q8pair != 2 && k % 64 == 0 && ((uintptr_t)w & 3) == 0 &&
           act_lds_bytes(k) + (size_t)k + 16 <= c->lds_limit;
}

int launch(jl_ctx* c, const char* name, unsigned gx, unsigned gy, unsigned block, unsigned lds,
           hipStream_t st, void** params, unsigned gz = 1) {
    auto it = c->fn.find(name);
    if (it == c->fn.end()) return fail(c, JL_ERR_ARG, "kernel %s is not in the code object", name);
    if (call_dry_run(c)) return JL_OK;
    HIP_TRY(c, H->ModuleLaunchKernel(it->second, gx, gy, gz, block, 1, 1, lds, st, params, nullptr));
    c->launches++;
    return JL_OK;
}

// Grows a context-owned device buffer.  Growing frees the old one, which kernels enqueued by
// earlier calls -- on the context's stream or on any stream a caller passed -- may still
// read, so the whole device is waited for first.  Never reached once the buffer is large
// enough (jl_reserve, jl_reserve_shape).
int grow(jl_ctx* c, void** buf, size_t* have, size_t need) {
    if (*have >= need) return JL_OK;
    if (call_no_alloc(c)) {
        // a call that must not allocate: the next piece of the static array, or an error.  (A
        // workspace asked for a second time with a larger size gets a new, larger piece: the
        // one it had stays taken until the call ends.)
        const size_t off = (g_call.static_used + 255) & ~(size_t)255;
        if (off + need > c->static_scratch_bytes)
            return fail(c, JL_ERR_NOMEM, "this shape needs %zu bytes of workspace on top of %zu already carved; the static "
                        "scratch holds %zu", need, off, c->static_scratch_bytes);
        *buf = (char*)c->static_scratch + off;
        *have = need;
        g_call.static_used = off + need;
        return JL_OK;
    }
    if (*buf) {
        HIP_TRY(c, H->DeviceSynchronize());
        HIP_TRY(c, H->Free(*buf));
    }
    *buf = nullptr;
    *have = 0;
    HIP_TRY(c, H->Malloc(buf, need));
    *have = need;
    return JL_OK;
}

// Shape checks shared by every matvec entry point.  Returns JL_OK, JL_DECLINED or an error.
int matvec_check(jl_ctx* c, int type, int nrows, int k, const TypeInfo** ti_out) {
    const TypeInfo* ti = type_info(type);
    if (!ti) return JL_DECLINED;
    if (nrows <= 0 || k <= 0) return fail(c, JL_ERR_ARG, "matvec: nrows=%d k=%d", nrows, k);
    if (k % ti->block_elems != 0) return JL_DECLINED;
    size_t lds = (size_t)k + (size_t)(k / 32) * 4 + (size_t)(k / 16) * 4;
    if (lds > c->lds_limit) return JL_DECLINED;  // activation does not fit LDS
    if ((size_t)(k / ti->block_elems) * ti->block_bytes > 0x7fffffffu) return JL_DECLINED;
    *ti_out = ti;
    return JL_OK;
}

int matvec_launch(jl_ctx* c, float* out, int type, const void* w, const float* x, const int8_t* q,
                  const float* as, const float* s16, int nrows, int k, hipStream_t st, float* resid = nullptr,
                  float alpha = 0.f, const float* resid_gate = nullptr) {
    const TypeInfo* ti = nullptr;
    int rc = matvec_check(c, type, nrows, k, &ti);
    if (rc != JL_OK) return rc;
    if (!out || !w) return fail(c, JL_ERR_ARG, "matvec: null operand");
    if (x && !aligned16(x)) return JL_DECLINED;
    if (!x && (!q || !as || !s16)) return fail(c, JL_ERR_ARG, "matvec: no activation");
    if (q && !aligned16(q)) return JL_DECLINED;
    if (type == JL_TYPE_Q4_K && !aligned16(w)) return JL_DECLINED;
    if (((uintptr_t)w & 1) != 0) return JL_DECLINED;

    // Shape choice, from sweeps on MI355X: one row per wavefront; a matrix with at
    // most sixteen rows per CU runs one 16-wavefront workgroup per CU (the CU
    // quantizes x once), larger ones a persistent grid of two 12-wavefront
    // workgroups per CU that stride over the row groups.
    int rpw = c->tune.rpw, block = c->tune.block;
    if (rpw <= 0 || resid || !x) rpw = 1;   // (the kernels with the residual add or a quantized activation: one row a wavefront)
    if (rpw != 1 && rpw != 2 && rpw != 4) return fail(c, JL_ERR_ARG, "matvec: rpw=%d", rpw);
    const bool small = nrows <= 16 * c->num_cu;
    // (Q4_K 14336 x 4096: one 16-wavefront workgroup a CU 8.1 us, two of twelve 8.6)
    const bool one_per_cu = small || type == JL_TYPE_Q6_K || type == JL_TYPE_Q4_K;
    if (block <= 0) block = one_per_cu ? 1024 : 768;
    if (block % 64 != 0 || block > 1024) return fail(c, JL_ERR_ARG, "matvec: block=%d", block);
    const bool pair = q8_pair_form(c, type, w, k);
    if (block > matvec_max_block(type, rpw, pair)) block = matvec_max_block(type, rpw, pair);
    const int rows_per_block = (block / 64) * rpw;
    long groups = ((long)nrows + rows_per_block - 1) / rows_per_block;
    long grid = c->tune.grid > 0 ? c->tune.grid : (long)c->num_cu * (type == JL_TYPE_Q4_K && !small ? 1 : 2);
    if (grid > groups) grid = groups;
    if (grid < 1) grid = 1;

    MatVecArgs a;
    a.out = out;
    a.w = (const uint8_t*)w;
    a.x = x;
    a.q = q;
    a.as = as;
    a.s16 = s16;
    a.nrows = nrows;
    a.k = k;
    a.row_bytes = (k / ti->block_elems) * ti->block_bytes;
    a.per = c->act_window / 32;
    a.nwaves = block / 64;
    a.ngroups = (int)grid;
    a.resid = resid; a.alpha = alpha; a.resid_gate = resid ? resid_gate : nullptr;
    const int xpre = c->tune.xpre == 1 || c->tune.xpre == 4 ? c->tune.xpre : (k / 4 > 2 * block ? 4 : 1);   // three groups a thread and more
    char name[64];
    snprintf(name, sizeof name, "jl_matvec_%s_r%d%s%s", pair ? "q8_0p" : ti->tag, rpw, !x ? "_pq" : xpre == 4 ? "_x4" : "",
             resid ? "_res" : "");
    void* params[] = {&a};
    unsigned lds = (unsigned)(act_lds_bytes(k) + (pair ? (size_t)k + 16 : 0));
    return launch(c, name, (unsigned)grid, 1, (unsigned)block, lds, st, params);
}

// m matrices of one type in one launch (kernels/matvec.h, matvec_multi_body).
// types: null when every matrix is of `type`; else the type of each (the mixed-type kernel).
int matvec_multi_launch(jl_ctx* c, int type, int m, float* const* outs, const void* const* ws, const int* rows,
                        const float* x, size_t xstride, const float* x2, float* resid, float alpha, int k,
                        hipStream_t st, const float* norm_w = nullptr, float norm_eps = 0.f,
                        float* norm_out = nullptr, const int* types = nullptr, const float* resid_gate = nullptr) {
    if (m < 1 || m > JL_MAX_MULTI) return fail(c, JL_ERR_ARG, "matvec multi: %d matrices", m);
    const TypeInfo* ti = nullptr;
    const TypeInfo* tis[JL_MAX_MULTI];
    int max_rows = 0;
    for (int i = 0; i < m; i++) {
        const int t = types ? types[i] : type;
        int rc = matvec_check(c, t, rows[i], k, &ti);
        if (rc != JL_OK) return rc;
        tis[i] = ti;
        if (!outs[i] || !ws[i]) return fail(c, JL_ERR_ARG, "matvec multi: null operand");
        if (t == JL_TYPE_Q4_K && !aligned16(ws[i])) return JL_DECLINED;
        if (((uintptr_t)ws[i] & 1) != 0) return JL_DECLINED;
        if (rows[i] > max_rows) max_rows = rows[i];
    }
    if (!x || !aligned16(x) || (x2 && !aligned16(x2)) || (xstride % 4) != 0) return JL_DECLINED;
    if ((norm_w && !aligned16(norm_w)) || (norm_out && !aligned16(norm_out))) return JL_DECLINED;
    MatVecMultiArgs a;
    memset(&a, 0, sizeof a);
    for (int i = 0; i < m; i++) {
        a.out[i] = outs[i];
        a.w[i] = (const uint8_t*)ws[i];
        a.nrows[i] = rows[i];
        a.type[i] = types ? types[i] : type;
        a.row_bytes_of[i] = (k / tis[i]->block_elems) * tis[i]->block_bytes;
    }
    a.x = x; a.x2 = x2; a.resid = resid; a.alpha = alpha; a.resid_gate = resid ? resid_gate : nullptr;
    a.xstride = xstride;
    a.norm_w = norm_w; a.norm_eps = norm_eps; a.norm_out = norm_out;
    a.k = k; a.row_bytes = (k / ti->block_elems) * ti->block_bytes; a.per = c->act_window / 32;
    // sixteen wavefronts a workgroup, one row each; about two workgroups per CU over all
    // the matrices, never more row groups than the tallest matrix has
    const int nwaves = 16;
    long groups = ((long)max_rows + nwaves - 1) / nwaves;
    long gx = (2L * c->num_cu + m - 1) / m;
    if (gx > groups) gx = groups;
    if (gx < 1) gx = 1;
    a.nwaves = nwaves; a.ngroups = (int)gx;
    const int xpre = c->tune.xpre == 1 || c->tune.xpre == 4 ? c->tune.xpre : (k / 4 > 2 * nwaves * 64 ? 4 : 1);
    char name[64];
    bool pair = !types;
    for (int i = 0; i < m && pair; i++) pair = q8_pair_form(c, type, ws[i], k);
    // "matvec.act_split" = 1: a gated activation shared by the group's matrices is formed and
    // quantized once, by the quantizer kernel, and the matvec stages the int8 copy (the same
    // values, bit for bit).  Not the default: the extra launch costs what it saves (Q6_K
    // 4096 x 14336 over silu(gate) * up: 15.2 us against 14.4 with every workgroup forming it).
    const bool split_act = x2 && !types && !norm_w && xstride == 0 && c->tune.act_split == 1;
    // A single matrix with nothing in front of its quantizer but (perhaps) that activation is the
    // plain decode matvec with the residual add riding on it: its kernel carries no norm or gate
    // code and keeps every row loop in registers (Q6_K 4096 x 14336: 10.8 against 12.2 us).
    if (m == 1 && !types && !norm_w && (!x2 || split_act) && c->tune.act_split != 3) {
        const int8_t* q = nullptr;
        const float *as = nullptr, *s16 = nullptr;
        if (x2) {
            const size_t o_as = ((size_t)k + 255) & ~(size_t)255, o_s16 = o_as + (((size_t)(k / 32) * 4 + 255) & ~(size_t)255);
            int rc = grow(c, &c->act_ws, &c->act_ws_bytes, o_s16 + (size_t)(k / 16) * 4);
            if (rc != JL_OK) return rc;
            int8_t* qq = (int8_t*)c->act_ws;
            float* asw = (float*)((char*)c->act_ws + o_as);
            float* s16w = (float*)((char*)c->act_ws + o_s16);
            int per = c->act_window / 32;
            void* qp[] = {(void*)&x, (void*)&qq, (void*)&asw, (void*)&s16w, (void*)&k, (void*)&per, (void*)&x2};
            rc = launch(c, "jl_quantize_act", (unsigned)((k / 4 + 255) / 256), 1, 256, 0, st, qp);
            if (rc != JL_OK) return rc;
            q = qq; as = asw; s16 = s16w;
        }
        return matvec_launch(c, outs[0], type, ws[0], x2 ? nullptr : x, q, as, s16, rows[0], k, st, resid, alpha,
                             resid_gate);
    }
    if (split_act) {
        const size_t o_as = ((size_t)k + 255) & ~(size_t)255, o_s16 = o_as + (((size_t)(k / 32) * 4 + 255) & ~(size_t)255);
        int rc = grow(c, &c->act_ws, &c->act_ws_bytes, o_s16 + (size_t)(k / 16) * 4);
        if (rc != JL_OK) return rc;
        int8_t* q = (int8_t*)c->act_ws;
        float* as = (float*)((char*)c->act_ws + o_as);
        float* s16 = (float*)((char*)c->act_ws + o_s16);
        int per = c->act_window / 32;
        void* qp[] = {(void*)&x, (void*)&q, (void*)&as, (void*)&s16, (void*)&k, (void*)&per, (void*)&x2};
        rc = launch(c, "jl_quantize_act", (unsigned)((k / 4 + 255) / 256), 1, 256, 0, st, qp);
        if (rc != JL_OK) return rc;
        a.x = nullptr; a.x2 = nullptr; a.q = q; a.as = as; a.s16 = s16;
        snprintf(name, sizeof name, "jl_matvec_multi_%s_q%s", pair ? "q8_0p" : ti->tag, resid ? "_res" : "");
        void* params[] = {&a};
        unsigned lds = (unsigned)(act_lds_bytes(k) + (pair ? (size_t)k + 16 : 0));
        return launch(c, name, (unsigned)gx, (unsigned)m, nwaves * 64, lds, st, params);
    }
    if (types) snprintf(name, sizeof name, "jl_matvec_segments");
    else snprintf(name, sizeof name, "jl_matvec_multi_%s%s%s", pair ? "q8_0p" : ti->tag, xpre == 4 ? "_x4" : "",
                  resid ? "_res" : "");
    void* params[] = {&a};
    // (+ 16 to round the staging area up, + JL_NORM_LDS_BYTES for the RMSNorm's partial sums)
    unsigned lds = (unsigned)(act_lds_bytes(k) + (pair ? (size_t)k + 16 : 0) + 16 + 160);
    return launch(c, name, (unsigned)gx, (unsigned)m, nwaves * 64, lds, st, params);
}

int ensure_stage(jl_ctx* c, void** buf, size_t* have, size_t need) { return grow(c, buf, have, need); }

// Applies the ranges jl_forget queued: every device copy keyed inside one of them is
// unlinked and freed.  Called with c->mu held, before a residency lookup.
void drain_forget(jl_ctx* c) {
    std::vector<std::pair<uintptr_t, uintptr_t>> todo;
    {
        std::lock_guard<std::mutex> g(c->forget_mu);
        todo.swap(c->pending_forget);
    }
    for (const auto& r : todo)
        for (auto it = c->resident.begin(); it != c->resident.end();) {
            const uintptr_t k0 = (uintptr_t)it->first;
            if (k0 >= r.first && k0 < r.second) {
                if (!c->no_device) (void)H->Free(it->second.dev);
                it = c->resident.erase(it);
            } else {
                ++it;
            }
        }
}

// Device copy of host weight bytes, keyed on the host pointer.
int resident_weight(jl_ctx* c, const void* w, size_t bytes, void** dev) {
    auto it = c->resident.find(w);
    if (it != c->resident.end() && it->second.bytes == bytes) {
        *dev = it->second.dev;
        return JL_OK;
    }
    if (it != c->resident.end()) {
        HIP_TRY(c, H->Free(it->second.dev));
        c->resident.erase(it);
    }
    void* d = nullptr;
    HIP_TRY(c, H->Malloc(&d, bytes));
    hipError_t e = H->Memcpy(d, w, bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)H->Free(d);
        return fail(c, JL_ERR_HIP, "weight upload: %s", H->GetErrorString(e));
    }
    c->resident[w] = Resident{d, bytes};
    *dev = d;
    return JL_OK;
}

int ws_ensure(jl_ctx* c, void** buf, size_t* have, size_t need);
int moe_matvec_launch(jl_ctx* c, float* out0, float* out1, int type, const void* bank0, const void* bank1,
                      const float* x, const float* x2, const uint32_t* src, const uint32_t* start,
                      int n_expert, int ncols, int nrows, int k, hipStream_t st,
                      const jl_packed_bank* pb0 = nullptr, const jl_packed_bank* pb1 = nullptr);

// plane banks of a mixture: from this many columns an expert (on average) the matrix-core tile
// per expert takes over from the dot-product form ("moe.form" = 1 / 4 forces one)
constexpr long kMoePlaneTileCols = 14;
constexpr int kGemmTile = 128;         // tokens and rows per workgroup (kernels/gemm_q4k.h)
constexpr int kGemmStride = 152;       // f16 per stage row
constexpr unsigned gemm_lds_bytes(int rows) {   // two weight stages, row scales, token scales
    return 2u * rows * kGemmStride * 2u + 2u * 2u * rows * 4u + 2u * kGemmTile * 4u;
}
constexpr unsigned kGemmLdsBytes = gemm_lds_bytes(128);
constexpr size_t kGemmAStageBytes = 9 * 1024;  // per 32 tokens and stage: nine fragments of 64 lanes x 16 B

size_t gemm_ws_need(int ntok, int k) {
    size_t tok_pad = ((size_t)ntok + 255) / 256 * 256;   // the widest token tile of any form
    size_t nsb = (size_t)k / 256;
    return nsb * 2 * (tok_pad / 32) * kGemmAStageBytes + nsb * tok_pad * 4;
}

int gemm_ws_ensure(jl_ctx* c, size_t need) { return grow(c, &c->gemm_ws, &c->gemm_ws_bytes, need); }

constexpr size_t kGemmW16StageVecs = 1152;   // JL_GEMM_W16_STAGE_VECS
constexpr unsigned kGemmW16LdsBytes = 2u * 1152u * 16u + 2u * kGemmTile * 4u;

// Two-pass form: expand the weights into f16 fragments once, then the matrix kernel.
int gemm_q4k_w16_launch(jl_ctx* c, float* out, const void* w, const uint16_t* bq, const float* da, int nrows,
                        int k, int ntok, int tok_pad, hipStream_t st) {
    const int nsb = k / 256;
    const int nrt = (nrows + 63) / 64, nrows_pad = nrt * 64, ntt = tok_pad / kGemmTile;
    const size_t w16_bytes = (size_t)nrt * 2 * nsb * kGemmW16StageVecs * 16;
    const size_t need = w16_bytes + (size_t)nsb * nrows_pad * 8;
    int rcw = grow(c, &c->w16_ws, &c->w16_ws_bytes, need);
    if (rcw != JL_OK) return rcw;
    float* wsc = (float*)((char*)c->w16_ws + w16_bytes);
    GemmW16PrepArgs pa;
    pa.w = (const uint8_t*)w; pa.w16 = c->w16_ws; pa.wsc = wsc;
    pa.nrows = nrows; pa.nrows_pad = nrows_pad; pa.k = k; pa.row_bytes = nsb * 144;
    void* pp[] = {&pa};
    int rc = launch(c, "jl_gemm_w16_prep_q4k", (unsigned)nsb, (unsigned)(nrows_pad / 32), 256, 0, st, pp);
    if (rc != JL_OK) return rc;
    GemmW16Args ga;
    ga.out = out; ga.w16 = c->w16_ws; ga.wsc = wsc; ga.bq = bq; ga.da = da;
    ga.nrows = nrows; ga.nrows_pad = nrows_pad; ga.k = k; ga.ntok = ntok; ga.tok_pad = tok_pad;
    ga.ntt = ntt; ga.nrt = nrt;
    void* gp[] = {&ga};
    const unsigned groups = (unsigned)((nrt + 7) / 8 * 8) * (unsigned)ntt;
    return launch(c, "jl_gemm_q4k_w16", groups, 1, 256, kGemmW16LdsBytes, st, gp);
}

// Q4_K prefill GEMM on the f16 matrix cores; operands are device pointers.  Forms (tuning
// key "gemm.form", 0 = choose): 1 = 128-token x 64-row tiles, weights dequantized in the
// kernel; 2 = 256-token x 128-row tiles, a wavefront across all 128 rows (least L1 traffic
// per matrix instruction, for grids that still fill the chip); 3 = weights expanded once
// per call into f16 fragments, then 128 x 64 tiles; 6 = 128 x 64 tiles that walk the whole of K,
// its halves on two groups of four wavefronts (grids of half a round up to one round of the chip).
struct PlaneRef {
    const uint32_t *qs, *d, *sc;
    int row, stride;
};

constexpr int kGemmWideTok = 256;
// JL_GEMM_K2_LDS_BYTES: two groups of (two weight stages, minimum columns, row scales, token scales)
constexpr unsigned kGemmK2LdsBytes = 2u * (2u * 64u * 136u * 2u + 2u * 64u * 24u * 2u + 2u * 64u * 2u * 4u + 2u * 128u * 4u);
constexpr unsigned kGemmWideLdsBytes = 2u * 128u * 136u * 2u + 2u * 128u * 24u * 2u + 2u * 128u * 2u * 4u + 2u * kGemmWideTok * 4u;   // JL_GEMM_WIDE_LDS_BYTES

// Few tokens, or a grid of at most a round and a half of 32-row workgroups: the forms that
// take a lane's operand words straight from GGUF rows (no plane form of them exists).
bool gemm_q4k_few_applies(const jl_ctx* c, int nrows, int k, int ntok) {
    const int form = c->tune.gemm_form;
    if ((size_t)nrows * (size_t)(k / 256) * 144 >= ((size_t)1 << 32)) return false;
    if ((form == 0 || form == 4) && ntok <= 64) return true;
    const long few32_groups = (long)((nrows + 31) / 32) * ((ntok + 63) / 64);
    return ((form == 0 && 2 * few32_groups <= 3L * c->num_cu) || (form == 5 && ntok <= 1024)) && ntok > 64;
}

// pl: the weights as packed planes (w unused): the tiled forms read them where they lie.  The
// caller has checked that gemm_q4k_few_applies() is false.
int gemm_q4k_launch(jl_ctx* c, float* out, const void* w, const float* x, int nrows, int k, int ntok,
                    hipStream_t st, const PlaneRef* pl = nullptr) {
    int form = c->tune.gemm_form;
    if (pl && form == 3) form = 0;
    if (!pl && (form == 0 || form == 4) && ntok <= 64 && (size_t)nrows * (size_t)(k / 256) * 144 < ((size_t)1 << 32)) {
        // few tokens: 16-row workgroups that split K over their wavefronts, one launch after
        // the activation prep (kernels/gemm_q4k.h, "few tokens")
        const int tok_pad = (ntok + 31) / 32 * 32, nsb = k / 256, nt = (ntok + 15) / 16;
        int rc = gemm_ws_ensure(c, gemm_ws_need(tok_pad, k));
        if (rc != JL_OK) return rc;
        uint16_t* bq = (uint16_t*)c->gemm_ws;
        float* da = (float*)((char*)c->gemm_ws + (size_t)nsb * 2 * (tok_pad / 32) * kGemmAStageBytes);
        GemmPrepArgs pa;
        pa.x = x; pa.bq = bq; pa.da = da; pa.ntok = ntok; pa.tok_pad = tok_pad; pa.k = k;
        void* pp[] = {&pa};
        rc = launch(c, "jl_gemm_prep_q4k_w16", (unsigned)nsb, (unsigned)(tok_pad / 32), 1024, 0, st, pp);
        if (rc != JL_OK) return rc;
        GemmArgs ga;
        ga.out = out; ga.w = (const uint8_t*)w; ga.bq = bq; ga.da = da;
        ga.nrows = nrows; ga.k = k; ga.ntok = ntok; ga.tok_pad = tok_pad; ga.row_bytes = nsb * 144;
        ga.out_stride = nrows; ga.sb_per = 0;
        void* gp[] = {&ga};
        char name[32];
        snprintf(name, sizeof name, "jl_gemm_q4k_few_t%d", nt);
        return launch(c, name, (unsigned)((nrows + 15) / 16), 1, 512, 0, st, gp);
    }
    const long few32_groups = (long)((nrows + 31) / 32) * ((ntok + 63) / 64);
    if (!pl && ((form == 0 && 2 * few32_groups <= 3L * c->num_cu) || (form == 5 && ntok <= 1024)) && ntok > 64 &&
        (size_t)nrows * (size_t)(k / 256) * 144 < ((size_t)1 << 32)) {
        // some more tokens, few enough rows: the same scheme on 32-row x 64-token workgroups,
        // one to a CU, while the grid is at most a round and a half (4096 rows: up to 192
        // tokens; measured against the tiled forms, 128 tokens x 4096 rows 24.6 -> 16.5 us;
        // at 14336 rows the tiled forms win)
        const int tok_pad = (ntok + 63) / 64 * 64, nsb = k / 256;
        int rc = gemm_ws_ensure(c, gemm_ws_need(tok_pad, k));
        if (rc != JL_OK) return rc;
        uint16_t* bq = (uint16_t*)c->gemm_ws;
        float* da = (float*)((char*)c->gemm_ws + (size_t)nsb * 2 * (tok_pad / 32) * kGemmAStageBytes);
        GemmPrepArgs pa;
        pa.x = x; pa.bq = bq; pa.da = da; pa.ntok = ntok; pa.tok_pad = tok_pad; pa.k = k;
        void* pp[] = {&pa};
        rc = launch(c, "jl_gemm_prep_q4k_w16", (unsigned)nsb, (unsigned)(tok_pad / 32), 1024, 0, st, pp);
        if (rc != JL_OK) return rc;
        GemmArgs ga;
        ga.out = out; ga.w = (const uint8_t*)w; ga.bq = bq; ga.da = da;
        ga.nrows = nrows; ga.k = k; ga.ntok = ntok; ga.tok_pad = tok_pad; ga.row_bytes = nsb * 144;
        ga.out_stride = nrows; ga.sb_per = 0;
        void* gp[] = {&ga};
        return launch(c, "jl_gemm_q4k_few32", (unsigned)((nrows + 31) / 32), (unsigned)(tok_pad / 64), 512, 0, st, gp);
    }
    if (form == 4 || form == 5) form = 0;   // outside the few-token forms' range
    const bool k2_fits = (k / 256) % 4 == 0 && kGemmK2LdsBytes <= c->lds_limit;
    if (form == 0 && k2_fits) {
        // 128 x 64 tiles over the whole of K: from half a round of the chip up to one round nothing
        // has to be cut along K and added afterwards (measured against the forms below, us:
        // 512 tokens x 4096 rows 32.0 against 37.9, 384 x 4096 29.4 against 35.9, 128 x 14336
        // 27.9 against 36.2, 256 x 4096 26.5 against 27.7; two rounds and more go to the wide tile)
        const long k2_groups = (long)((ntok + kGemmTile - 1) / kGemmTile) * ((nrows + 63) / 64);
        if (k2_groups <= c->num_cu && 2 * k2_groups >= c->num_cu) form = 6;
    }
    if (form == 0) {
        const long wide_groups = (long)((ntok + kGemmWideTok - 1) / kGemmWideTok) * ((nrows + 127) / 128);
        // from a quarter of the CUs on: a smaller grid is widened along K below (measured
        // against the 64-row tiles: 1024 tokens x 4096 rows 56 against 62 us, 512 x 4096 38 against 40)
        // (not for a last token tile that is mostly padding: 128 tokens x 14336 rows 40 against 45 us)
        const bool padded = (ntok % kGemmWideTok) != 0 && (ntok % kGemmWideTok) <= kGemmWideTok / 2 && ntok < 2 * kGemmWideTok;
        form = 4 * wide_groups >= 3 * (long)c->num_cu || (4 * wide_groups >= (long)c->num_cu && !padded) ? 2 : 1;
    }
    if (form == 2 && kGemmWideLdsBytes > c->lds_limit) form = 1;
    if (form == 6 && !k2_fits) form = 1;
    // the opt-in folded-scale form (kernels/gemm_q4k_fold.h): asked for with "gemm.fold" = 1,
    // and only for a matrix whose scales jl_fold_admit_dev has checked
    bool fold = false;
    if (c->tune.gemm_fold == 1 && form == 2 && !pl && 2u * 128u * 136u * 2u <= c->lds_limit) {
        std::lock_guard<std::mutex> g(c->forget_mu);
        auto it = c->fold_ok.find((uintptr_t)w);
        fold = it != c->fold_ok.end() && it->second.first == nrows && it->second.second == k;
    }
    const int tile = form == 2 ? kGemmWideTok : kGemmTile;
    const int tok_pad = (ntok + tile - 1) / tile * tile;
    const int nsb = k / 256;
    int rc = gemm_ws_ensure(c, gemm_ws_need(tok_pad, k));
    if (rc != JL_OK) return rc;
    uint16_t* bq = (uint16_t*)c->gemm_ws;
    float* da = (float*)((char*)c->gemm_ws + (size_t)nsb * 2 * (tok_pad / 32) * kGemmAStageBytes);
    GemmPrepArgs pa;
    pa.x = x; pa.bq = bq; pa.da = da; pa.ntok = ntok; pa.tok_pad = tok_pad; pa.k = k;
    void* pp[] = {&pa};
    // sixteen wavefronts a workgroup: the chain of tokens a wavefront quantizes one after the other
    // is the kernel's length (whole matmul, 512 tokens x 4096 rows: 41.0 -> 39.7 us; 2048 tokens:
    // 87.1 -> 83.4; "gemm.prep" = 4 asks for four wavefronts)
    const bool prep16 = c->tune.gemm_prep != 4;
    // (the plane kernels take the activations in the planes' K order: their own prep)
    rc = launch(c, fold ? "jl_gemm_prep_q4k_fold" : pl ? "jl_gemm_prep_q4k_planes" : prep16 ? "jl_gemm_prep_q4k_w16" : "jl_gemm_prep_q4k",
                (unsigned)nsb, (unsigned)(tok_pad / 32), fold || pl || prep16 ? 1024 : 256, 0, st, pp);
    if (rc != JL_OK) return rc;
    if (form == 3) return gemm_q4k_w16_launch(c, out, w, bq, da, nrows, k, ntok, tok_pad, st);
    GemmArgs ga;
    if (pl) { ga.pqs = pl->qs; ga.pd = pl->d; ga.psc = pl->sc; ga.prow0 = pl->row; ga.pstride = pl->stride; }
    ga.out = out; ga.w = (const uint8_t*)w; ga.bq = bq; ga.da = da;
    ga.nrows = nrows; ga.k = k; ga.ntok = ntok; ga.tok_pad = tok_pad; ga.row_bytes = nsb * 144;
    ga.out_stride = nrows; ga.sb_per = 0;
    void* gp[] = {&ga};
    if (fold) {
        // four wavefronts a workgroup, two workgroups a CU, from a full round of the chip on;
        // eight below (measured, us: 2048 tokens x 14336 rows 238 against 251; 1024 x 4096
        // 59.7 against 55.1; a round or so, 2048 x 4096 and 512 x 14336, the same)
        const long groups = (long)(tok_pad / kGemmWideTok) * ((nrows + 127) / 128);
        const bool w8 = c->tune.gemm_fold_waves == 8 || (c->tune.gemm_fold_waves != 4 && groups < (long)c->num_cu);
        return launch(c, w8 ? "jl_gemm_q4k_fold_wide" : "jl_gemm_q4k_fold_wide4", (unsigned)(tok_pad / kGemmWideTok),
                      (unsigned)((nrows + 127) / 128), w8 ? 512 : 256, 2u * 128u * 136u * 2u, st, gp);   // JL_GEMM_FOLD_LDS_BYTES
    }
    if (form == 6)   // 128 x 64 tiles over the whole of K, the K halves on two groups of wavefronts
        return launch(c, pl ? "jl_gemm_q4k_k2_planes" : "jl_gemm_q4k_k2", (unsigned)(tok_pad / kGemmTile), (unsigned)((nrows + 63) / 64), 512,
                      kGemmK2LdsBytes, st, gp);
    int rows_left = nrows;
    if (form == 2) {
        // One workgroup per CU: a grid of f full rounds and a last round at most half full
        // leaves half the chip idle for a whole round.  The rows of that last round go to the
        // 128 x 64 tiles instead (two workgroups per CU), which fill the chip once more.
        const long ntt = tok_pad / kGemmWideTok, nrt = (nrows + 127) / 128;
        const long full = ntt * nrt / c->num_cu, rem = ntt * nrt - full * c->num_cu;
        long nrt_wide = nrt;
        if (c->tune.gemm_form == 0 && full >= 1 && rem > 0 && 2 * rem <= c->num_cu) nrt_wide = full * c->num_cu / ntt;
        ga.nrows = nrt_wide == nrt ? nrows : (int)(nrt_wide * 128);
        // a grid of at most half the CUs is widened along K, partial slabs added in order
        int wsplit = c->tune.gemm_split > 0 ? c->tune.gemm_split : (c->tune.gemm_form == 0 ? (int)(c->num_cu / (ntt * nrt)) : 1);
        if (wsplit > 8) wsplit = 8;
        if (wsplit > nsb) wsplit = nsb;
        if (wsplit > 1) {
            const int per = (nsb + wsplit - 1) / wsplit;
            wsplit = (nsb + per - 1) / per;   // no empty split
        }
        if (wsplit > 1 && nrt_wide == nrt) {
            const size_t n = (size_t)ntok * nrows;
            rc = ws_ensure(c, &c->mx_ws, &c->mx_ws_bytes, n * wsplit * 4);
            if (rc != JL_OK) return rc;
            ga.out = (float*)c->mx_ws; ga.sb_per = (nsb + wsplit - 1) / wsplit;
            rc = launch(c, pl ? "jl_gemm_q4k_wide_planes" : "jl_gemm_q4k_wide", (unsigned)ntt, (unsigned)nrt, 512,
                        kGemmWideLdsBytes, st, gp, (unsigned)wsplit);
            if (rc != JL_OK) return rc;
            SumPartsArgs sa;
            sa.out = out; sa.part = (const float*)c->mx_ws; sa.n = n; sa.nsplit = wsplit;
            void* sp[] = {&sa};
            return launch(c, "jl_sum_parts", (unsigned)((n + 255) / 256), 1, 256, 0, st, sp);
        }
        rc = launch(c, pl ? "jl_gemm_q4k_wide_planes" : "jl_gemm_q4k_wide", (unsigned)ntt, (unsigned)nrt_wide, 512,
                    kGemmWideLdsBytes, st, gp);
        rows_left = nrows - ga.nrows;
        if (rc != JL_OK || rows_left == 0) return rc;
        if (pl) ga.prow0 += ga.nrows;
        else ga.w += (size_t)ga.nrows * ga.row_bytes;
        ga.out += ga.nrows;
        ga.nrows = rows_left;
    }
    // 64-row workgroups, two to a CU, unless asked for the 128-row form
    const int rows = c->tune.gemm_rows == 128 && !pl ? 128 : 64;
    const char* const r64 = pl ? "jl_gemm_q4k_r64_planes" : "jl_gemm_q4k_r64";
    if (rows == 64 && rows_left == nrows) {
        // a grid that leaves most of the chip idle (few tokens) is widened along K
        const long groups = (long)(tok_pad / kGemmTile) * ((nrows + 63) / 64);
        int nsplit = c->tune.gemm_split > 0 ? c->tune.gemm_split
                     : (c->tune.gemm_form == 0 && groups <= c->num_cu ? (int)(2 * c->num_cu / groups) : 1);
        if (nsplit > 8) nsplit = 8;
        if (nsplit > nsb) nsplit = nsb;
        if (nsplit > 1) {
            const int per = (nsb + nsplit - 1) / nsplit;
            nsplit = (nsb + per - 1) / per;   // no empty split
            const size_t n = (size_t)ntok * nrows;
            rc = ws_ensure(c, &c->mx_ws, &c->mx_ws_bytes, n * nsplit * 4);
            if (rc != JL_OK) return rc;
            ga.out = (float*)c->mx_ws; ga.sb_per = per;
            rc = launch(c, r64, (unsigned)(tok_pad / kGemmTile), (unsigned)((nrows + 63) / 64), 256,
                        gemm_lds_bytes(64), st, gp, (unsigned)nsplit);
            if (rc != JL_OK) return rc;
            SumPartsArgs sa;
            sa.out = out; sa.part = (const float*)c->mx_ws; sa.n = n; sa.nsplit = nsplit;
            void* sp[] = {&sa};
            return launch(c, "jl_sum_parts", (unsigned)((n + 255) / 256), 1, 256, 0, st, sp);
        }
    }
    return launch(c, rows == 128 ? "jl_gemm_q4k_r128" : r64, (unsigned)(tok_pad / kGemmTile),
                  (unsigned)((rows_left + rows - 1) / rows), rows == 128 ? 512 : 256, gemm_lds_bytes(rows), st, gp);
}

// Q6_K prefill GEMM on the f16 matrix cores (kernels/gemm_q6k.h): 128-token x 64-row tiles,
// the Q4_K form's activation prep; a grid that leaves most of the chip idle is widened along
// K and the partial slabs are added in order.
constexpr unsigned kGemm6LdsBytes = 2u * 64u * kGemmStride * 2u;   // JL_GEMM6_LDS_BYTES

int gemm_q6k_launch(jl_ctx* c, float* out, const void* w, const float* x, int nrows, int k, int ntok,
                    hipStream_t st) {
    const int tok_pad = (ntok + kGemmTile - 1) / kGemmTile * kGemmTile, nsb = k / 256;
    int rc = gemm_ws_ensure(c, gemm_ws_need(tok_pad, k));
    if (rc != JL_OK) return rc;
    uint16_t* bq = (uint16_t*)c->gemm_ws;
    float* da = (float*)((char*)c->gemm_ws + (size_t)nsb * 2 * (tok_pad / 32) * kGemmAStageBytes);
    GemmPrepArgs pa;
    pa.x = x; pa.bq = bq; pa.da = da; pa.ntok = ntok; pa.tok_pad = tok_pad; pa.k = k;
    void* pp[] = {&pa};
    rc = launch(c, "jl_gemm_prep_q4k_w16", (unsigned)nsb, (unsigned)(tok_pad / 32), 1024, 0, st, pp);
    if (rc != JL_OK) return rc;
    GemmArgs ga;
    ga.out = out; ga.w = (const uint8_t*)w; ga.bq = bq; ga.da = da;
    ga.nrows = nrows; ga.k = k; ga.ntok = ntok; ga.tok_pad = tok_pad; ga.row_bytes = nsb * 210;
    ga.out_stride = nrows; ga.sb_per = 0;
    void* gp[] = {&ga};
    const long groups = (long)(tok_pad / kGemmTile) * ((nrows + 63) / 64);
    int nsplit = c->tune.gemm_split > 0 ? c->tune.gemm_split : (groups <= c->num_cu ? (int)(2 * c->num_cu / groups) : 1);
    if (nsplit > 8) nsplit = 8;
    if (nsplit > nsb) nsplit = nsb;
    if (nsplit > 1) {
        const int per = (nsb + nsplit - 1) / nsplit;
        nsplit = (nsb + per - 1) / per;   // no empty split
        const size_t n = (size_t)ntok * nrows;
        rc = ws_ensure(c, &c->mx_ws, &c->mx_ws_bytes, n * nsplit * 4);
        if (rc != JL_OK) return rc;
        ga.out = (float*)c->mx_ws; ga.sb_per = per;
        rc = launch(c, "jl_gemm_q6k_r64", (unsigned)(tok_pad / kGemmTile), (unsigned)((nrows + 63) / 64),
                    256, kGemm6LdsBytes, st, gp, (unsigned)nsplit);
        if (rc != JL_OK) return rc;
        SumPartsArgs sa;
        sa.out = out; sa.part = (const float*)c->mx_ws; sa.n = n; sa.nsplit = nsplit;
        void* sp[] = {&sa};
        return launch(c, "jl_sum_parts", (unsigned)((n + 255) / 256), 1, 256, 0, st, sp);
    }
    return launch(c, "jl_gemm_q6k_r64", (unsigned)(tok_pad / kGemmTile), (unsigned)((nrows + 63) / 64), 256,
                  kGemm6LdsBytes, st, gp);
}

// Q8_0, Q6_K and Q4_K prefill GEMM with the activation window of 32 (kernels/gemm_w32.h): its own
// prep (fragments in the order of the byte unpack, a token scale per 32), 128-token x 64-row
// tiles, K split in stages of 128 (Q6_K: whole super-blocks) for small grids.
constexpr unsigned gemm32_lds_bytes(int planes) {   // JL_GEMM32_LDS_BYTES
    return (unsigned)planes * 64u * kGemmStride * 2u + 2u * 64u * 4u * 4u + 2u * 4u * kGemmTile * 4u;
}

int gemm_w32_launch(jl_ctx* c, float* out, int type, const void* w, const float* x, int nrows, int k, int ntok,
                    hipStream_t st) {
    const bool q6 = type == JL_TYPE_Q6_K, q4 = type == JL_TYPE_Q4_K;
    const char* kernel = q6 ? "jl_gemm_q6k_w32" : q4 ? "jl_gemm_q4k_w32" : "jl_gemm_q8_0_w32";
    const unsigned lds = gemm32_lds_bytes(q6 ? 2 : 1);
    const int tok_pad = (ntok + kGemmTile - 1) / kGemmTile * kGemmTile, nstage = k / 128;
    const size_t bq_bytes = (size_t)nstage * (tok_pad / 32) * 8 * 1024, da_bytes = (size_t)(k / 32) * tok_pad * 4;
    int rc = gemm_ws_ensure(c, bq_bytes + (q4 ? 2 : 1) * da_bytes);
    if (rc != JL_OK) return rc;
    uint16_t* bq = (uint16_t*)c->gemm_ws;
    float* da = (float*)((char*)c->gemm_ws + bq_bytes);
    GemmPrepArgs pa;
    pa.x = x; pa.bq = bq; pa.da = da; pa.ntok = ntok; pa.tok_pad = tok_pad; pa.k = k;
    if (q4) pa.dsum = (float*)((char*)da + da_bytes);   // the minimums meet d_a * block sums
    void* pp[] = {&pa};
    rc = launch(c, "jl_gemm_prep_w32", (unsigned)((k + 255) / 256), (unsigned)(tok_pad / 32), 256, 0, st, pp);
    if (rc != JL_OK) return rc;
    GemmArgs ga;
    ga.out = out; ga.w = (const uint8_t*)w; ga.bq = bq; ga.da = da;
    ga.nrows = nrows; ga.k = k; ga.ntok = ntok; ga.tok_pad = tok_pad;
    ga.row_bytes = q6 ? (k / 256) * 210 : q4 ? (k / 256) * 144 : (k / 32) * 34;
    ga.out_stride = nrows; ga.sb_per = 0; ga.dsum = pa.dsum;
    void* gp[] = {&ga};
    const long groups = (long)(tok_pad / kGemmTile) * ((nrows + 63) / 64);
    const int unit = q6 || q4 ? 2 : 1, nunit = nstage / unit;   // stages a split is made of
    int nsplit = c->tune.gemm_split > 0 ? c->tune.gemm_split : (groups <= c->num_cu ? (int)(2 * c->num_cu / groups) : 1);
    if (nsplit > 8) nsplit = 8;
    if (nsplit > nunit) nsplit = nunit;
    if (nsplit > 1) {
        const int per = (nunit + nsplit - 1) / nsplit;
        nsplit = (nunit + per - 1) / per;   // no empty split
        const size_t n = (size_t)ntok * nrows;
        rc = ws_ensure(c, &c->mx_ws, &c->mx_ws_bytes, n * nsplit * 4);
        if (rc != JL_OK) return rc;
        ga.out = (float*)c->mx_ws; ga.sb_per = per * unit;
        rc = launch(c, kernel, (unsigned)(tok_pad / kGemmTile), (unsigned)((nrows + 63) / 64), 256, lds, st, gp,
                    (unsigned)nsplit);
        if (rc != JL_OK) return rc;
        SumPartsArgs sa;
        sa.out = out; sa.part = (const float*)c->mx_ws; sa.n = n; sa.nsplit = nsplit;
        void* sp[] = {&sa};
        return launch(c, "jl_sum_parts", (unsigned)((n + 255) / 256), 1, 256, 0, st, sp);
    }
    return launch(c, kernel, (unsigned)(tok_pad / kGemmTile), (unsigned)((nrows + 63) / 64), 256, lds, st, gp);
}

// out [ntok][nrows] = x [ntok][k] W^T on device operands: the matrix-core GEMM where it
// applies, else one fused matvec launch per token (same values, token by token).
int matmul_launch(jl_ctx* c, float* out, int type, const void* w, const float* x, int nrows, int k,
                  int ntok, hipStream_t st) {
    const TypeInfo* ti = nullptr;
    int rc = matvec_check(c, type, nrows, k, &ti);
    if (rc != JL_OK) return rc;
    if (!out || !w || !x || ntok <= 0) return fail(c, JL_ERR_ARG, "matmul: bad operand");
    if (!aligned16(x) || (k % 4) != 0) return JL_DECLINED;
    const bool gemm = type == JL_TYPE_Q4_K && c->act_window == 256 && ntok >= c->gemm_min_tok &&
                      aligned16(w) && ntok <= 65535 * 4 && kGemmLdsBytes <= c->lds_limit;
    if (gemm) return gemm_q4k_launch(c, out, w, x, nrows, k, ntok, st);
    if (type == JL_TYPE_Q6_K && c->act_window == 256 && ntok >= c->gemm_min_tok && c->tune.gemm_form != 9 &&
        ((uintptr_t)w & 1) == 0 && ntok <= 65535 * 4 && (nrows + 63) / 64 <= 65535 && kGemm6LdsBytes <= c->lds_limit)
        return gemm_q6k_launch(c, out, w, x, nrows, k, ntok, st);   // ("gemm.form" = 9: token by token)
    // Q8_0, a handful of tokens: the grouped dot-product kernel with the tokens as the columns
    // of a single group streams the rows once and beats the 128-token tile (14336 x 4096:
    // 2 tokens 17.4 against 21.7 us token by token, 3 tokens 18.6 against 35.2 for the tile, 8 tokens
    // 26.9 against 34.3, 12 tokens 41.8 against 34.5; Q6_K rows are too long for that kernel: 62 us at 3)
    if (type == JL_TYPE_Q8_0 && ntok >= 2 && ntok <= 8 && c->tune.gemm_form == 0 && aligned16(w) &&
        (size_t)nrows * ti->block_bytes * (k / ti->block_elems) % 2 == 0) {
        rc = moe_matvec_launch(c, out, nullptr, type, w, nullptr, x, nullptr, nullptr, c->one_group + 2 * ntok, 1, ntok,
                               nrows, k, st);
        if (rc != JL_DECLINED) return rc;
    }
    if ((type == JL_TYPE_Q8_0 || type == JL_TYPE_Q6_K || type == JL_TYPE_Q4_K) && c->act_window == 32 &&
        ntok >= c->gemm_min_tok && c->tune.gemm_form != 9 && k % 128 == 0 && ((uintptr_t)w & 1) == 0 && ntok <= 65535 * 4 &&
        (nrows + 63) / 64 <= 65535 && gemm32_lds_bytes(2) <= c->lds_limit)
        return gemm_w32_launch(c, out, type, w, x, nrows, k, ntok, st);
    for (int t = 0; t < ntok; t++) {
        rc = matvec_launch(c, out + (size_t)t * nrows, type, w, x + (size_t)t * k, nullptr, nullptr,
                           nullptr, nrows, k, st);
        if (rc != JL_OK) return rc;
    }
    return JL_OK;
}

int ws_ensure(jl_ctx* c, void** buf, size_t* have, size_t need) { return grow(c, buf, have, need); }

// Words of the three planes of an nrows x k matrix (jit/gpu/kernels/pack.go:580-621).
bool packed_words(int type, size_t nrows, int k, size_t* nq, size_t* nd, size_t* nsc) {
    if (k <= 0 || nrows == 0) return false;
    switch (type) {
    case JL_TYPE_Q4_K:
        if (k % 256) return false;
        *nq = nrows * (size_t)(k / 32) * 4; *nd = nrows * (size_t)(k / 256); *nsc = *nd * 3;
        return true;
    case JL_TYPE_Q6_K:
        if (k % 256) return false;
        *nq = nrows * (size_t)(k / 16) * 3; *nd = nrows * (size_t)(k / 256); *nsc = nrows * (size_t)(k / 64);
        return true;
    case JL_TYPE_Q8_0:
        if (k % 32) return false;
        *nq = nrows * (size_t)(k / 32) * 8; *nd = (size_t)(k / 32) * ((nrows + 1) / 2); *nsc = 0;
        return true;
    case JL_TYPE_MXFP4:   // DSlots 4: an exponent byte a row, four rows a word (pack.go:543-575)
        if (k % 32) return false;
        *nq = nrows * (size_t)(k / 32) * 4; *nd = (size_t)(k / 32) * ((nrows + 3) / 4); *nsc = 0;
        return true;
    }
    return false;
}

int packed_check(jl_ctx* c, int type, const PlaneRef& pl, int nrows, int k, const TypeInfo** ti) {
    *ti = type_info(type);
    if (!*ti) return JL_DECLINED;
    if (nrows <= 0 || k <= 0 || pl.row < 0 || pl.stride <= 0)
        return fail(c, JL_ERR_ARG, "packed: nrows=%d k=%d row=%d stride=%d", nrows, k, pl.row, pl.stride);
    if ((long)pl.row + nrows > pl.stride)
        return fail(c, JL_ERR_ARG, "packed: rows %d..%d outside a buffer of %d rows", pl.row, pl.row + nrows, pl.stride);
    if (k % (*ti)->block_elems != 0) return JL_DECLINED;
    if (!pl.qs || !pl.d || (type != JL_TYPE_Q8_0 && !pl.sc)) return fail(c, JL_ERR_ARG, "packed: null plane");
    if (((uintptr_t)pl.qs | (uintptr_t)pl.d | (uintptr_t)pl.sc) & 3) return JL_DECLINED;
    return JL_OK;
}

int packed_matvec_launch(jl_ctx* c, float* out, int type, const PlaneRef& pl, const float* x,
                         const int8_t* q, const float* as, const float* s16, int nrows, int k,
                         hipStream_t st) {
    const TypeInfo* ti = nullptr;
    int rc = packed_check(c, type, pl, nrows, k, &ti);
    if (rc != JL_OK) return rc;
    if (!out) return fail(c, JL_ERR_ARG, "packed matvec: null out");
    if (x && !aligned16(x)) return JL_DECLINED;
    if (!x && (!q || !as || !s16)) return fail(c, JL_ERR_ARG, "packed matvec: no activation");
    if (q && ((uintptr_t)q & 3)) return JL_DECLINED;
    // Rows per wavefront: the widest run that still gives three CUs in four a
    // workgroup (from sweeps: 224 workgroups of 64-row runs beat 448 of 32-row runs).
    int rw = c->tune.packed_rw;
    if (rw <= 0) {
        rw = 64;
        while (rw > 16 && (nrows + rw - 1) / rw < c->num_cu * 3 / 4) rw >>= 1;
    }
    if (rw != 16 && rw != 32 && rw != 64) return fail(c, JL_ERR_ARG, "packed matvec: rw=%d", rw);
    const int nchunks = (k + 255) / 256;
    // sixteen-row runs: eight wavefronts a workgroup, two workgroups a CU (measured against sixteen,
    // us: Q4_K 4096 x 4096 4.87 against 5.06, Q6_K 4096 x 14336 14.46 against 14.69)
    int nw = c->tune.packed_block > 0 ? c->tune.packed_block / 64 : rw == 16 ? 8 : 16;
    if (nw > nchunks) nw = nchunks;
    if (nw < 1 || nw > 16) return fail(c, JL_ERR_ARG, "packed matvec: block=%d", nw * 64);
    PackedMatVecArgs a;
    a.out = out; a.qs = pl.qs; a.d = pl.d; a.sc = pl.sc;
    a.x = x; a.q = q; a.as = as; a.s16 = s16;
    a.nrows = nrows; a.k = k; a.row0 = pl.row; a.stride = pl.stride; a.per = c->act_window / 32;
    a.nwaves = nw; a.ngroups = (nrows + rw - 1) / rw;
    a.x2 = nullptr; a.resid = nullptr; a.alpha = 0.f; a.norm_out = nullptr; a.norm_eps = 0.f;
    char name[64];
    snprintf(name, sizeof name, "jl_matvec_packed_%s%s_w%d", x ? "" : "q8_", ti->tag, rw);
    void* params[] = {&a};
    return launch(c, name, (unsigned)((nrows + rw - 1) / rw), 1, (unsigned)(nw * 64),
                  (unsigned)(nw * (384 + 65 * 4)), st, params);  // JL_PK_LDS_BYTES
}

// m packed matvecs of one type and shape in one launch (grid.y = matrix): each with its
// own planes and first row, reading x + j * xstride; up gates the activation.
int packed_matvec_multi_launch(jl_ctx* c, int type, int m, float* const* outs, const PlaneRef* pls,
                               const float* x, size_t xstride, const float* up, float* resid, float alpha,
                               const float* resid_gate, const float* norm_w, float norm_eps, float* norm_out,
                               int nrows, int k, hipStream_t st) {
    if (m < 1 || m > JL_MAX_MULTI) return fail(c, JL_ERR_ARG, "packed multi: %d matrices", m);
    // the norm precedes gate and up, the gated activation precedes down: never both
    if (norm_w && (up || !aligned16(norm_w) || (norm_out && !aligned16(norm_out)))) return JL_DECLINED;
    const TypeInfo* ti = nullptr;
    for (int j = 0; j < m; j++) {
        int rc = packed_check(c, type, pls[j], nrows, k, &ti);
        if (rc != JL_OK) return rc;
        if (!outs[j]) return fail(c, JL_ERR_ARG, "packed multi: null out");
        if (pls[j].stride != pls[0].stride) return JL_DECLINED;
    }
    if (!x || !aligned16(x) || (up && !aligned16(up)) || (xstride % 4) != 0) return JL_DECLINED;
    // rows per wavefront: the widest run that still gives three CUs in four a workgroup,
    // counting every matrix's row groups
    int rw = c->tune.packed_rw;
    if (rw <= 0) {
        rw = 64;
        while (rw > 16 && (long)m * ((nrows + rw - 1) / rw) < c->num_cu * 3 / 4) rw >>= 1;
    }
    if (rw != 16 && rw != 32 && rw != 64) return fail(c, JL_ERR_ARG, "packed multi: rw=%d", rw);
    const int nchunks = (k + 255) / 256;
    // sixteen-row runs: eight wavefronts a workgroup, two workgroups a CU (measured against sixteen,
    // us: Q4_K 4096 x 4096 4.87 against 5.06, Q6_K 4096 x 14336 14.46 against 14.69)
    int nw = c->tune.packed_block > 0 ? c->tune.packed_block / 64 : rw == 16 ? 8 : 16;
    if (nw > nchunks) nw = nchunks;
    if (nw < 1 || nw > 16) return fail(c, JL_ERR_ARG, "packed multi: block=%d", nw * 64);
    PackedMultiArgs a;
    memset(&a, 0, sizeof a);
    for (int j = 0; j < m; j++) {
        a.out[j] = outs[j]; a.qs[j] = pls[j].qs; a.d[j] = pls[j].d; a.sc[j] = pls[j].sc; a.row0[j] = pls[j].row;
    }
    a.x = x; a.x2 = up; a.xstride = xstride; a.resid = resid; a.alpha = alpha;
    a.resid_gate = resid ? resid_gate : nullptr;
    a.norm_w = norm_w; a.norm_eps = norm_eps; a.norm_out = norm_w ? norm_out : nullptr;
    a.nrows = nrows; a.k = k; a.stride = pls[0].stride; a.per = c->act_window / 32;
    a.nwaves = nw; a.ngroups = (nrows + rw - 1) / rw;
    char name[64];
    snprintf(name, sizeof name, "jl_matvec_packed_multi_%s%s_w%d", up ? "act_" : norm_w ? "norm_" : "", ti->tag, rw);
    void* params[] = {&a};
    return launch(c, name, (unsigned)a.ngroups, (unsigned)m, (unsigned)(nw * 64), (unsigned)(nw * (384 + 65 * 4)), st,
                  params);   // JL_PK_LDS_BYTES
}

// MXFP4 planes (QS and D only): rows row .. row+nrows of a buffer of `stride` rows.
int mx_planes_check(jl_ctx* c, const PlaneRef& pl, int nrows, int k) {
    if (nrows <= 0 || k <= 0 || pl.row < 0 || pl.stride <= 0)
        return fail(c, JL_ERR_ARG, "mxfp4 planes: nrows=%d k=%d row=%d stride=%d", nrows, k, pl.row, pl.stride);
    if ((long)pl.row + nrows > pl.stride)
        return fail(c, JL_ERR_ARG, "mxfp4 planes: rows %d..%d outside a buffer of %d rows", pl.row, pl.row + nrows,
                    pl.stride);
    if (!pl.qs || !pl.d) return fail(c, JL_ERR_ARG, "mxfp4 planes: null plane");
    if (k % 32 != 0 || k / 32 > 65535 || (((uintptr_t)pl.qs | (uintptr_t)pl.d) & 3)) return JL_DECLINED;
    return JL_OK;
}

int unpack_launch(jl_ctx* c, int type, const PlaneRef& pl, int nrows, int k, void* dst, hipStream_t st) {
    UnpackArgs a;
    a.dst = (uint8_t*)dst; a.qs = pl.qs; a.d = pl.d; a.sc = pl.sc;
    a.nrows = nrows; a.k = k; a.row0 = pl.row; a.stride = pl.stride;
    void* params[] = {&a};
    if (type == JL_TYPE_Q8_0 || type == JL_TYPE_MXFP4)
        return launch(c, type == JL_TYPE_Q8_0 ? "jl_unpack_q8_0" : "jl_unpack_mxfp4", (unsigned)((nrows + 255) / 256),
                      (unsigned)(k / 32), 256, 0, st, params);
    return launch(c, type == JL_TYPE_Q6_K ? "jl_unpack_q6k" : "jl_unpack_q4k", (unsigned)((nrows + 255) / 256),
                  (unsigned)(k / 256), 256, 0, st, params);
}

int packed_matmul_launch(jl_ctx* c, float* out, int type, const PlaneRef& pl, const float* x, int nrows,
                         int k, int ntok, hipStream_t st) {
    const TypeInfo* ti = nullptr;
    int rc = packed_check(c, type, pl, nrows, k, &ti);
    if (rc != JL_OK) return rc;
    if (!out || !x || ntok <= 0) return fail(c, JL_ERR_ARG, "packed matmul: bad operand");
    if (!aligned16(x) || (k % 4) != 0) return JL_DECLINED;
    // the matrix-core forms read GGUF rows: the planes are turned back into rows in a workspace
    const bool gemm = type == JL_TYPE_Q4_K && c->act_window == 256 && ntok >= c->gemm_min_tok &&
                      ntok <= 65535 * 4 && kGemmLdsBytes <= c->lds_limit && k / 256 <= 65535;
    const bool gemm6 = type == JL_TYPE_Q6_K && c->act_window == 256 && ntok >= c->gemm_min_tok &&
                       c->tune.gemm_form != 9 && ntok <= 65535 * 4 && (nrows + 63) / 64 <= 65535 &&
                       kGemm6LdsBytes <= c->lds_limit && k / 256 <= 65535;
    const bool gemm32 = (type == JL_TYPE_Q8_0 || type == JL_TYPE_Q6_K || type == JL_TYPE_Q4_K) && c->act_window == 32 &&
                        ntok >= c->gemm_min_tok && c->tune.gemm_form != 9 && k % 128 == 0 && ntok <= 65535 * 4 &&
                        (nrows + 63) / 64 <= 65535 && gemm32_lds_bytes(2) <= c->lds_limit && k / 32 <= 65535;
    // Q4_K with the k-quant window: the tiled forms read the planes where they lie; only the
    // few-token forms, which take a lane's operand words straight from GGUF rows, restore rows first
    if (gemm && c->tune.gemm_planes != 2 && !gemm_q4k_few_applies(c, nrows, k, ntok) && (size_t)pl.stride * 4 < ((size_t)1 << 31))
        return gemm_q4k_launch(c, out, nullptr, x, nrows, k, ntok, st, &pl);
    if (gemm || gemm6 || gemm32) {
        rc = ws_ensure(c, &c->unpack_ws, &c->unpack_ws_bytes, (size_t)nrows * (size_t)(k / ti->block_elems) * ti->block_bytes);
        if (rc != JL_OK) return rc;
        rc = unpack_launch(c, type, pl, nrows, k, c->unpack_ws, st);
        if (rc != JL_OK) return rc;
        if (gemm32) return gemm_w32_launch(c, out, type, c->unpack_ws, x, nrows, k, ntok, st);
        return gemm ? gemm_q4k_launch(c, out, c->unpack_ws, x, nrows, k, ntok, st)
                    : gemm_q6k_launch(c, out, c->unpack_ws, x, nrows, k, ntok, st);
    }
    for (int t = 0; t < ntok; t++) {
        rc = packed_matvec_launch(c, out + (size_t)t * nrows, type, pl, x + (size_t)t * k, nullptr, nullptr,
                                  nullptr, nrows, k, st);
        if (rc != JL_OK) return rc;
    }
    return JL_OK;
}

// pb0 / pb1: the banks as packed planes (bank0 / bank1 unused then): the per-expert tile kernel
// reads an expert's sheet where it lies in the bank's pages.
int moe_matvec_launch(jl_ctx* c, float* out0, float* out1, int type, const void* bank0, const void* bank1,
                      const float* x, const float* x2, const uint32_t* src, const uint32_t* start,
                      int n_expert, int ncols, int nrows, int k, hipStream_t st, const jl_packed_bank* pb0,
                      const jl_packed_bank* pb1) {
    const TypeInfo* ti = nullptr;
    int rc = matvec_check(c, type, nrows, k, &ti);
    if (rc != JL_OK) return rc;
    const bool planes = pb0 != nullptr;
    if (!out0 || (!planes && !bank0) || !x || !start || n_expert <= 0 || ncols <= 0)
        return fail(c, JL_ERR_ARG, "moe matvec: bad operand");
    if (planes) {
        if ((pb1 == nullptr) != (out1 == nullptr)) return fail(c, JL_ERR_ARG, "moe matvec: second matrix needs both bank and out");
        for (const jl_packed_bank* b : {pb0, pb1}) {
            if (!b) continue;
            if (!b->qs || !b->d || !b->sc || b->stride <= 0) return fail(c, JL_ERR_ARG, "moe matvec: null plane");
            if ((((uintptr_t)b->qs | (uintptr_t)b->d | (uintptr_t)b->sc) & 3) || (b->sheet_bytes & 3)) return JL_DECLINED;
            // an expert's rows must lie inside a plane set: its own sheet, or its range of the bank's
            if (b->sheet_bytes ? b->stride < nrows : (long)b->stride < (long)n_expert * nrows)
                return fail(c, JL_ERR_ARG, "moe matvec: plane sets of %d rows do not hold %d experts x %d rows", b->stride,
                            n_expert, nrows);
            if (b->sheet_bytes != pb0->sheet_bytes || b->stride != pb0->stride) return JL_DECLINED;   // one layout a launch
        }
        // plane sheets are served by the tile form (Q4_K, the k-quant window)
        if (type != JL_TYPE_Q4_K || c->act_window != 256) return JL_DECLINED;
        if ((size_t)pb0->stride * 4 >= ((size_t)1 << 31)) return JL_DECLINED;
    } else if ((bank1 == nullptr) != (out1 == nullptr)) {
        return fail(c, JL_ERR_ARG, "moe matvec: second matrix needs both bank and out");
    }
    if (!aligned16(x) || (x2 && !aligned16(x2)) || k % 256 != 0 || n_expert > 65535 || ncols > 65535) return JL_DECLINED;
    if (!planes && (!aligned16(bank0) || (bank1 && !aligned16(bank1)))) return JL_DECLINED;
    const int row_bytes = (k / ti->block_elems) * ti->block_bytes;
    const size_t sheet = (size_t)nrows * row_bytes;
    if (type == JL_TYPE_Q4_K ? sheet % 16 != 0 : sheet % 2 != 0) return JL_DECLINED;
    // Q4_K with the k-quant activation window can also run on the matrix cores (tuning
    // "moe.form" = 2: groups of 32 columns, a wavefront to itself; 3: groups of 16, the weights
    // decoded in registers, below; 4: the prefill GEMM's tile).  Their vector work does not grow
    // with the number of columns.  Measured at the 128-expert shape, top-8 (router + gate + up +
    // down + combine, whole block, us; forms 1 / 2 / 3 with groups of 16 / 3 with groups of 32 / 4):
    //   16 rows 73 / 155 / 85 / - / -       64 rows 133 / 210 / 110 / - / -     128 rows 191 / 223 / 130 / 137 / 302
    //   192 rows - / 232 / 171 / 147 / 309  256 rows 333 / 238 / 187 / 157 / 315  512 rows - / 301 / 281 / 243 / 352
    //   1024 rows - / 426 / 489 / 372 / 400 1280 rows - / 501 / 577 / 475 / 435   2048 rows - / 709 / 831 / 639 / 623
    // so form 3 takes over from two columns an expert on average (groups of 32 from ten) and form 4
    // from 72; form 2 is left to "moe.form" = 2.
    // Q6_K sheets (the down projections of a model whose other experts are Q4_K) have forms 1, 3
    // and 4 (the Q6_K GEMM's tile); where form 3 does not apply (K too long for LDS) the tile takes
    // over from "moe.q6k_cols" columns an expert on average, default 12.
    // Form 3: groups of sixteen columns on the 16 x 16 x 32 matrix instruction, the weights decoded
    // in registers straight into its operand (Q4_K GGUF sheets or packed planes, Q6_K GGUF sheets, the k-quant window; the group's
    // fragments for the whole of K sit in LDS).  Its steady state runs at the rate of a plain read;
    // the library picks it from two (over planes three) columns an expert on average up to 72, while the
    // fragments take at most half a CU's LDS (K <= 2304); "moe.form" = 3 forces it wherever they fit.
    {
        const int nsb = k / 256;
        const size_t frag16 = (size_t)nsb * JL_MOE_G16_LDS_WORDS * 4;   // a token tile's fragments
        const size_t lds16 = frag16 + 16;                               // and the tile counter
        const size_t nslots16 = (size_t)ncols / 16 + (size_t)n_expert + 1;
        const bool q6k = type == JL_TYPE_Q6_K;   // (GGUF sheets only: plane sheets are Q4_K)
        const bool can16 = (type == JL_TYPE_Q4_K || (q6k && !planes)) && c->act_window == 256 && lds16 <= c->lds_limit &&
                           (size_t)nrows * row_bytes < ((size_t)1 << 32);
        // (Q6_K sheets: the decode is 4.5 vector instructions a weight, two matrix instructions a K-step,
        // and the kernel is bound by them: 62 us for the 2048 x 768 down projections of 128 experts at 64
        // rows where the dot-product kernel takes 58; with two token tiles a decoded word it costs the
        // same, so it is picked from six columns an expert, always in groups of 32: 128 rows 68 us against
        // 97, 256 rows 71 against 139 for the tile, 1024 rows 193 against 195)
        const bool pick16 = c->tune.moe_form == 0 && 2 * lds16 <= c->lds_limit &&
                            (long)ncols >= (q6k ? 6L : planes ? 3L : 2L) * n_expert && (long)ncols < (q6k ? 64L : 72L) * n_expert;
        if (can16 && (c->tune.moe_form == 3 || pick16)) {
            // up to eight columns an expert the matrix kernel quantizes them itself: no prep launch,
            // no workspace ("moe.group16" = 1 forces the prep kernel, 2 the fused form)
            const bool fused = c->tune.moe_g16 == 2 || (c->tune.moe_g16 == 0 && !q6k && (long)ncols <= 8L * n_expert);
            // from ten columns an expert groups of 32 (two token tiles, a decoded word meets both), so
            // that an expert of 17-32 columns reads its sheet once ("moe.group16" = 3 forces them)
            const bool two = !fused && 2 * frag16 + 16 <= c->lds_limit &&
                             (c->tune.moe_g16 == 3 || (c->tune.moe_g16 == 0 && (q6k || (long)ncols >= 10L * n_expert)));
            MoeG16PrepArgs pa;
            pa.ws = nullptr;
            if (!fused) {
                rc = ws_ensure(c, &c->moe_q_ws, &c->moe_q_ws_bytes, nslots16 * nsb * JL_MOE_G16_SB_WORDS * 4);
                if (rc != JL_OK) return rc;
                pa.x = x; pa.x2 = x2; pa.src = src; pa.start = start; pa.ws = (uint32_t*)c->moe_q_ws;
                pa.k = k; pa.n_expert = n_expert; pa.ncols = ncols;
                void* pp[] = {&pa};
                rc = launch(c, planes ? "jl_moe_g16_prep_planes" : q6k ? "jl_moe_g16_prep_q6k" : "jl_moe_g16_prep", (unsigned)((ncols + 3) / 4), 1,
                            256, 0, st, pp);
                if (rc != JL_OK) return rc;
            }
            MoeG16Args ga;
            ga.out[0] = out0; ga.out[1] = out1;
            ga.bank[0] = (const uint8_t*)bank0; ga.bank[1] = (const uint8_t*)bank1;
            ga.ws = pa.ws; ga.start = start;
            if (fused) { ga.x = x; ga.x2 = x2; ga.src = src; }
            ga.sheet_bytes = sheet; ga.nrows = nrows; ga.k = k; ga.row_bytes = row_bytes;
            if (planes) {
                const jl_packed_bank* pbs[2] = {pb0, pb1};
                for (int m = 0; m < (pb1 ? 2 : 1); m++) { ga.pqs[m] = pbs[m]->qs; ga.pd[m] = pbs[m]->d; ga.psc[m] = pbs[m]->sc; }
                ga.sheet_words = pb0->sheet_bytes / 4;
                ga.row_step = pb0->sheet_bytes ? 0 : nrows;
                ga.pstride = pb0->stride;
            }
            // One workgroup of eight wavefronts a CU (the same age on every SIMD, tiles handed out as
            // they get to them: two younger workgroups of four measured 4 % slower), so the grid runs
            // in rounds of CUs workgroups; among the splits of the rows into blocks the one with the
            // least rounds x tiles a wavefront, the fewest blocks among equals (every block fills LDS
            // anew).  Experts that can have a column: at most one a column.  "moe.waves" = 4: the
            // two-workgroup form.
            const int nmat = (planes ? pb1 != nullptr : bank1 != nullptr) ? 2 : 1, tiles = (nrows + 15) / 16;
            const int nwaves = !two && c->tune.moe_waves == 4 ? 4 : 8;
            const long wgs_cu = nwaves == 4 ? 2 : 1;
            const int sets = (tiles + nwaves - 1) / nwaves;
            const long n_act = std::min<long>(n_expert, ncols);
            int best_blocks = 1;
            long best_cost = -1;
            for (int nb = 1; nb <= sets && nb <= 64; nb++) {
                const long per_wave = (sets + nb - 1) / nb;
                const long rounds = ((long)nb * n_act * nmat + wgs_cu * c->num_cu - 1) / (wgs_cu * c->num_cu);
                const long cost = rounds * per_wave;
                if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_blocks = nb; }
            }
            if (c->tune.moe_shares > 0) best_blocks = std::min(c->tune.moe_shares, sets);
            ga.tiles_wg = (tiles + best_blocks - 1) / best_blocks;   // handed out inside the workgroup as its wavefronts get to them
            ga.blocks = (tiles + ga.tiles_wg - 1) / ga.tiles_wg;
            ga.nmat = nmat; ga.n_expert = n_expert; ga.nwaves = nwaves;
            const long grid = 8L * ((n_expert + 7) / 8) * ga.blocks * nmat;
            if (grid >= (1L << 31)) return JL_DECLINED;
            // super-blocks a step: all of a short row, else two (288 contiguous bytes a row; four
            // measured 10 % slower at K = 2048: twice the bytes in flight before the first step)
            // (over planes one: a lane's twelve loads of a super-block go to twelve planes, and more
            // of them in flight measured 5 % slower)
            int ch = planes ? 1 : (nsb <= 3 ? nsb : 2);
            if (c->tune.moe_chunk >= 1 && c->tune.moe_chunk <= 3) ch = std::min(c->tune.moe_chunk, nsb);
            char name[32];
            snprintf(name, sizeof name, "jl_moe_g16%s_%c%d", planes ? "p" : q6k ? "q6" : "", fused ? (x2 ? 'g' : 'f') : two ? 'd' : 'c', ch);
            void* gp[] = {&ga};
            return launch(c, name, (unsigned)grid, 1, (unsigned)(64 * nwaves), (unsigned)(two ? 2 * frag16 + 16 : lds16), st, gp);
        }
    }
    if (planes && c->tune.moe_form != 4 && (c->tune.moe_form == 1 || (long)ncols < kMoePlaneTileCols * n_expert)) {
        // few columns an expert: the dot-product form over planes (rows on lanes, a lane's share of a
        // chunk loaded once for all the expert's columns, the columns as scalar operands)
        if ((size_t)ncols * (k / 256) * 88 >= ((size_t)1 << 32)) return JL_DECLINED;   // 32-bit word offsets in the kernel
        // the columns quantized once, chunk by chunk: 88 words a (column, 256 elements)
        rc = ws_ensure(c, &c->moe_q_ws, &c->moe_q_ws_bytes, (size_t)ncols * (k / 256) * 88 * 4);
        if (rc != JL_OK) return rc;
        MoeQuantArgs qa;
        qa.x = x; qa.x2 = x2; qa.src = src;
        qa.q = nullptr; qa.as = nullptr; qa.s16 = nullptr; qa.chunked = (uint32_t*)c->moe_q_ws;
        qa.k = k; qa.per = c->act_window / 32;
        void* qparams[] = {&qa};
        rc = launch(c, "jl_moe_quant", (unsigned)((k / 4 + 255) / 256), (unsigned)ncols, 256, 0, st, qparams);
        if (rc != JL_OK) return rc;
        MoePlanesArgs a;
        const jl_packed_bank* pbs[2] = {pb0, pb1};
        const int nmat = pb1 ? 2 : 1;
        for (int m = 0; m < 2; m++) {
            a.out[m] = m == 0 ? out0 : out1;
            a.pqs[m] = m < nmat ? pbs[m]->qs : nullptr; a.pd[m] = m < nmat ? pbs[m]->d : nullptr;
            a.psc[m] = m < nmat ? pbs[m]->sc : nullptr;
        }
        a.chunked = qa.chunked; a.start = start;
        a.sheet_words = pb0->sheet_bytes / 4; a.row_step = pb0->sheet_bytes ? 0 : nrows; a.pstride = pb0->stride;
        a.nrows = nrows; a.k = k;
        a.nwaves = std::min(8, k / 256);
        void* params[] = {&a};
        return launch(c, "jl_moe_matvec_planes_q4k", (unsigned)((nrows + 63) / 64), (unsigned)n_expert, (unsigned)(a.nwaves * 64),
                      (unsigned)(a.nwaves * 8 * 256), st, params, (unsigned)nmat);   // JL_MOEP_TB columns a pass
    }
    const bool q6 = type == JL_TYPE_Q6_K;
    const long q6_cols = c->tune.moe_q6k_cols > 0 ? c->tune.moe_q6k_cols : 12;
    const bool many_cols = c->tune.moe_form == 0 && (long)ncols >= (q6 ? q6_cols : 10L) * n_expert;   // (Q4_K: 72 and more get here)
    if ((type == JL_TYPE_Q4_K || q6) && c->act_window == 256 &&
        (planes || c->tune.moe_form == 4 || many_cols || (!q6 && c->tune.moe_form == 2)) &&
        4u * 19968u <= c->lds_limit) {   // JL_MOEG_WAVE_LDS
        const int nslots = ncols / 32 + n_expert + 1, nsb = k / 256;
        const int tiles_max = ncols / 128 + n_expert;
        if (nslots > 65535) return JL_DECLINED;
        auto up256 = [](size_t v) { return (v + 255) & ~(size_t)255; };
        const size_t bq_bytes = (size_t)2 * nsb * nslots * kGemmAStageBytes;
        const size_t o_wl = bq_bytes + up256((size_t)nsb * nslots * 32 * 4);
        rc = ws_ensure(c, &c->moe_q_ws, &c->moe_q_ws_bytes, o_wl + (size_t)(4 + nslots + tiles_max) * 4);
        if (rc != JL_OK) return rc;
        // the work list of groups and tiles, from start[]
        MoeWorklistArgs wa;
        wa.start = start; wa.wl = (uint32_t*)((char*)c->moe_q_ws + o_wl);
        wa.n_expert = n_expert; wa.nslots = nslots;
        void* wp[] = {&wa};
        rc = launch(c, "jl_moe_worklist", 1, 1, 1024, 0, st, wp);
        if (rc != JL_OK) return rc;
        MoeGemmPrepArgs pa;
        pa.x = x; pa.x2 = x2; pa.src = src; pa.start = start; pa.wl = wa.wl;
        pa.bq = (uint16_t*)c->moe_q_ws; pa.da = (float*)((char*)c->moe_q_ws + bq_bytes);
        pa.k = k; pa.nslots = nslots;
        void* pp[] = {&pa};
        rc = launch(c, planes ? "jl_moe_gemm_prep_planes" : "jl_moe_gemm_prep", (unsigned)nsb, (unsigned)nslots, 256, 0, st, pp);
        if (rc != JL_OK) return rc;
        MoeGemmArgs ga;
        ga.out[0] = out0; ga.out[1] = out1;
        ga.bank[0] = (const uint8_t*)bank0; ga.bank[1] = (const uint8_t*)bank1;
        ga.bq = pa.bq; ga.da = pa.da; ga.start = start; ga.wl = wa.wl;
        ga.sheet_bytes = sheet; ga.nrows = nrows; ga.k = k; ga.row_bytes = row_bytes;
        ga.nslots = nslots; ga.nmat = (planes ? pb1 != nullptr : bank1 != nullptr) ? 2 : 1;
        if (planes) {
            const jl_packed_bank* pbs[2] = {pb0, pb1};
            for (int m = 0; m < ga.nmat; m++) { ga.pqs[m] = pbs[m]->qs; ga.pd[m] = pbs[m]->d; ga.psc[m] = pbs[m]->sc; }
            ga.sheet_words = pb0->sheet_bytes / 4;
            ga.row_step = pb0->sheet_bytes ? 0 : nrows;
            ga.pstride = pb0->stride;
        }
        void* gp[] = {&ga};
        const long rtiles = (nrows + 63) / 64;
        if (planes) {
            if (kGemmLdsBytes > c->lds_limit || (long)tiles_max * rtiles * ga.nmat >= (1L << 31)) return JL_DECLINED;
            const long work = (long)tiles_max * rtiles * ga.nmat;
            return launch(c, "jl_moe_gemm_r64_planes", (unsigned)std::min<long>(work, 2L * c->num_cu), 1, 256,
                          gemm_lds_bytes(64), st, gp);
        }
        if ((q6 || c->tune.moe_form == 4 || (c->tune.moe_form == 0 && (long)ncols >= 56L * n_expert)) &&
            kGemmLdsBytes <= c->lds_limit && n_expert <= 65535 && (long)tiles_max * rtiles * ga.nmat < (1L << 31)) {
            const long work = (long)tiles_max * rtiles * ga.nmat;
            const unsigned grid = (unsigned)std::min<long>(work, (q6 ? 3L : 2L) * c->num_cu);
            return launch(c, q6 ? "jl_moe_gemm_q6k_r64" : "jl_moe_gemm_r64", grid, 1, 256,
                          q6 ? kGemm6LdsBytes : gemm_lds_bytes(64), st, gp);
        }
        if (q6) return fail(c, JL_ERR_ARG, "moe matvec: %d experts x %ld row tiles do not fit the tile form", n_expert, rtiles);
        return launch(c, "jl_moe_gemm_q4k", (unsigned)((nrows + 255) / 256), (unsigned)nslots, 256, 4u * 19968u, st, gp,
                      (unsigned)ga.nmat);
    }
    if (planes) return JL_DECLINED;   // (no LDS for the tile form on this device)
    const int nslots = k / ti->slot_elems;
    // lanes per row: the width that leaves the fewest lanes without a slot (a row of 12 slots
    // on 16 lanes idles a quarter of them; on 4 lanes, three slots each, none); among equals
    // eight lanes, several slots a lane, measured best (sweeps at the 128-expert shape);
    // tuning "moe.lpr" overrides
    int lpr = 64, waste = 1 << 30;
    for (int cand : {8, 16, 4, 32, 64}) {
        const int w = (nslots + cand - 1) / cand * cand - nslots;
        if (w < waste) { waste = w; lpr = cand; }
    }
    {
        // (100 * a + b: a for rows of more than 16 slots, b for shorter ones)
        const int tl = c->tune.moe_lpr > 64 ? (nslots > 16 ? c->tune.moe_lpr / 100 : c->tune.moe_lpr % 100) : c->tune.moe_lpr;
        if (tl == 4 || tl == 8 || tl == 16 || tl == 32 || tl == 64) lpr = tl;
    }
    const size_t act = ((size_t)k + (size_t)(k / 32) * 4 + (size_t)(k / 16) * 4 + 15) & ~(size_t)15;
    const size_t lds = 8 * act;
    if (lds > c->lds_limit) return JL_DECLINED;

    // every column's activation, quantized once: q [ncols][k], as [ncols][k/32], s16 [ncols][k/16]
    auto up256 = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t o_as = up256((size_t)ncols * k), o_s16 = o_as + up256((size_t)ncols * (k / 32) * 4);
    rc = ws_ensure(c, &c->moe_q_ws, &c->moe_q_ws_bytes, o_s16 + up256((size_t)ncols * (k / 16) * 4));
    if (rc != JL_OK) return rc;
    char* qws = (char*)c->moe_q_ws;
    MoeQuantArgs qa;
    qa.x = x; qa.x2 = x2; qa.src = src;
    qa.q = (int8_t*)qws; qa.as = (float*)(qws + o_as); qa.s16 = (float*)(qws + o_s16);
    qa.k = k; qa.per = c->act_window / 32;
    void* qparams[] = {&qa};
    rc = launch(c, "jl_moe_quant", (unsigned)((k / 4 + 255) / 256), (unsigned)ncols, 256, 0, st, qparams);
    if (rc != JL_OK) return rc;

    MoeMatVecArgs a;
    a.out[0] = out0; a.out[1] = out1;
    a.bank[0] = (const uint8_t*)bank0; a.bank[1] = (const uint8_t*)bank1;
    a.q = qa.q; a.as = qa.as; a.s16 = qa.s16; a.start = start;
    a.sheet_bytes = sheet; a.nrows = nrows; a.k = k; a.row_bytes = row_bytes;
    // A workgroup of four wavefronts covers 4 * 2 * (64 / lpr) rows per step; at the kernel's
    // ~150 registers three such workgroups fill a CU's twelve wavefront slots, where one of
    // eight wavefronts leaves four empty (sweeps at the 128-expert, 64-row shape: 210 -> 150 us
    // for the block).  Row shares: about twelve workgroups per CU when every expert is in use,
    // each share at least one step.
    const int nmat = bank1 ? 2 : 1, nwaves = c->tune.moe_waves > 0 && c->tune.moe_waves <= 8 ? c->tune.moe_waves : 4;
    const int rows_per_step = nwaves * 2 * (64 / lpr);  // JL_MOE_U row groups per wavefront step
    int shares = c->tune.moe_shares;
    if (shares <= 0) {
        shares = (12 * c->num_cu + n_expert * nmat - 1) / (n_expert * nmat);
        const int most = (nrows + rows_per_step - 1) / rows_per_step;
        if (shares > most) shares = most;
    }
    if (shares < 1) shares = 1;
    if (shares > 65535) shares = 65535;
    a.nwaves = nwaves; a.shares = shares;
    char name[64];
    snprintf(name, sizeof name, "jl_moe_matvec_%s_l%d", ti->tag, lpr);
    void* params[] = {&a};
    return launch(c, name, (unsigned)shares, (unsigned)n_expert, nwaves * 64, (unsigned)lds, st, params, (unsigned)nmat);
}

}  // namespace

extern "C" {

int jl_ctx_create(jl_ctx** out, const jl_options* opts) {
    if (!out) return fail(nullptr, JL_ERR_ARG, "jl_ctx_create: null out");
    *out = nullptr;
    if (!H) {
        std::string why;
        H = hip_api(&why);
        if (!H) return fail(nullptr, JL_ERR_HIP, "%s", why.c_str());
    }
    jl_ctx* c = new (std::nothrow) jl_ctx;
    if (!c) return fail(nullptr, JL_ERR_NOMEM, "out of memory");
    c->device = opts ? opts->device : 0;
    c->act_window = (opts && opts->act_window) ? opts->act_window : 32;
    std::string path = (opts && opts->code_object) ? opts->code_object : default_code_object();

    auto bail = [&](int code, const std::string& msg) {
        g_create_error = msg;
        jl_ctx_destroy(c);
        return code;
    };
    if (c->act_window != 32 && c->act_window != 64 && c->act_window != 128 && c->act_window != 256)
        return bail(JL_ERR_ARG, "act_window must be 32, 64, 128 or 256");
    if (c->device < 0) {
        // no device: the host-side bookkeeping (residency keys, the forget queue, the lock)
        // works, every entry point that needs the GPU fails at its hipSetDevice
        c->no_device = true;
        *out = c;
        return JL_OK;
    }
    hipError_t e = H->SetDevice(c->device);
    if (e != hipSuccess) return bail(JL_ERR_HIP, std::string("hipSetDevice: ") + H->GetErrorString(e));
    hipDeviceProp_t prop;
    e = H->GetDeviceProperties(&prop, c->device);
    if (e != hipSuccess) return bail(JL_ERR_HIP, std::string("hipGetDeviceProperties: ") + H->GetErrorString(e));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return bail(JL_ERR_HIP, std::string("device is ") + prop.gcnArchName + ", this library is gfx950 only");
    c->num_cu = prop.multiProcessorCount;
    c->lds_limit = prop.sharedMemPerBlock;
    {
        // the static workspace's address on this device, looked up once per device with the
        // device current; a failure only disables the entry point that lives on it
        const char* why = "";
        if (jl_static_scratch_get(c->device, &c->static_scratch, &c->static_scratch_bytes, &why) != 0) {
            c->static_scratch = nullptr;
            c->static_scratch_bytes = 0;
            c->static_err = why;
        }
    }
    e = H->StreamCreate(&c->stream);
    if (e != hipSuccess) return bail(JL_ERR_HIP, std::string("hipStreamCreate: ") + H->GetErrorString(e));
    e = H->ModuleLoad(&c->module, path.c_str());
    if (e != hipSuccess)
        return bail(JL_ERR_HIP, "hipModuleLoad(" + path + "): " + H->GetErrorString(e));

    std::vector<std::string> names = {"jl_quantize_act", "jl_dequant", "jl_matvec_q4k_r1_pq", "jl_matvec_q4k_r1_pq_res", "jl_matvec_q8_0_r1_pq", "jl_matvec_q8_0_r1_pq_res", "jl_matvec_q6k_r1_pq", "jl_matvec_q6k_r1_pq_res", "jl_matvec_q8_0p_r1_pq", "jl_matvec_q8_0p_r1_pq_res", "jl_matvec_multi_q4k_res", "jl_matvec_multi_q4k_x4_res", "jl_matvec_multi_q4k_q_res", "jl_matvec_multi_q8_0_res", "jl_matvec_multi_q8_0_x4_res", "jl_matvec_multi_q8_0_q_res", "jl_matvec_multi_q6k_res", "jl_matvec_multi_q6k_x4_res", "jl_matvec_multi_q6k_q_res", "jl_matvec_multi_q8_0p_res", "jl_matvec_multi_q8_0p_x4_res", "jl_matvec_multi_q8_0p_q_res", "jl_matvec_q4k_r1_res", "jl_matvec_q4k_r1_x4_res", "jl_matvec_q8_0_r1_res", "jl_matvec_q8_0_r1_x4_res", "jl_matvec_q6k_r1_res", "jl_matvec_q6k_r1_x4_res", "jl_matvec_q8_0p_r1_res", "jl_matvec_q8_0p_r1_x4_res", "jl_matvec_q8_0p_r1", "jl_matvec_q8_0p_r2", "jl_matvec_q8_0p_r4", "jl_gemm_prep_q4k", "jl_gemm_prep_q4k_w16", "jl_gemm_q4k_r64", "jl_gemm_q6k_r64", "jl_gemm_prep_w32", "jl_gemm_q8_0_w32", "jl_gemm_q6k_w32", "jl_gemm_q4k_w32", "jl_gemm_q4k_r128", "jl_gemm_q4k_wide", "jl_gemm_prep_q4k_fold", "jl_gemm_q4k_fold_wide", "jl_gemm_q4k_fold_wide4", "jl_gemm_q4k_k2", "jl_gemm_q4k_k2_planes", "jl_gemm_prep_q4k_planes", "jl_gemm_q4k_r64_planes", "jl_gemm_q4k_wide_planes", "jl_gemm_w16_prep_q4k", "jl_gemm_q4k_w16", "jl_gemm_q4k_few_t1", "jl_gemm_q4k_few_t2", "jl_gemm_q4k_few_t3", "jl_gemm_q4k_few_t4", "jl_gemm_q4k_few32", "jl_moe_route", "jl_moe_route_g2", "jl_moe_route_g4", "jl_moe_logits", "jl_moe_logits_e8", "jl_moe_group", "jl_moe_group2", "jl_moe_group2_wide", "jl_moe_quant", "jl_moe_matvec_planes_q4k", "jl_moe_combine", "jl_moe_worklist", "jl_moe_gemm_prep", "jl_moe_gemm_prep_planes", "jl_moe_gemm_q4k", "jl_moe_g16_prep", "jl_moe_g16_prep_planes", "jl_moe_g16_prep_q6k", "jl_moe_g16_c1", "jl_moe_g16_c2", "jl_moe_g16_c3", "jl_moe_g16_f1", "jl_moe_g16_f2", "jl_moe_g16_f3", "jl_moe_g16_g1", "jl_moe_g16_g2", "jl_moe_g16_g3", "jl_moe_g16_d1", "jl_moe_g16_d2", "jl_moe_g16_d3", "jl_moe_g16p_c1", "jl_moe_g16p_c2", "jl_moe_g16p_c3", "jl_moe_g16p_f1", "jl_moe_g16p_f2", "jl_moe_g16p_f3", "jl_moe_g16p_g1", "jl_moe_g16p_g2", "jl_moe_g16p_g3", "jl_moe_g16p_d1", "jl_moe_g16p_d2", "jl_moe_g16p_d3", "jl_moe_g16q6_c1", "jl_moe_g16q6_c2", "jl_moe_g16q6_c3", "jl_moe_g16q6_f1", "jl_moe_g16q6_f2", "jl_moe_g16q6_f3", "jl_moe_g16q6_g1", "jl_moe_g16q6_g2", "jl_moe_g16q6_g3", "jl_moe_g16q6_d1", "jl_moe_g16q6_d2", "jl_moe_g16q6_d3", "jl_moe_gemm_r64", "jl_moe_gemm_r64_planes", "jl_moe_gemm_q6k_r64", "jl_mxfp4_prep", "jl_mxfp4_prep_few", "jl_mxfp4_few_t1", "jl_mxfp4_few_t2", "jl_mxfp4_few_t3", "jl_mxfp4_few_t4", "jl_mxfp4_gemm", "jl_mxfp4_gemm_r96", "jl_mxfp4_matvec", "jl_mxfp4_matvec1_b1", "jl_mxfp4_matvec1_b2", "jl_mxfp4_matvec1_b3", "jl_mxfp4_scaled_prep", "jl_mxfp4_scaled_gemm", "jl_mxfp4_planes_prep", "jl_mxfp4_planes_gemm", "jl_mxfp4_matvec_planes_r64", "jl_mxfp4_matvec_planes_r32", "jl_mxfp4_matvec_planes_r16", "jl_unpack_mxfp4", "jl_sum_parts", "jl_fill_u32", "jl_q4k_fold_range", "jl_probe_read", "jl_probe_empty", "jl_probe_wait", "jl_probe_mfma", "jl_probe_mfma_v5",
                                      "jl_pack_weights", "jl_unpack_q4k", "jl_unpack_q6k", "jl_unpack_q8_0"};
    for (const char* tag : {"q4k", "q8_0", "q6k"})
        for (int rw : {16, 32, 64})
            for (const char* form : {"", "q8_"})
                names.push_back(std::string("jl_matvec_packed_") + form + tag + "_w" + std::to_string(rw));
    for (const char* tag : {"q4k", "q8_0", "q6k"})
        for (int lpr : {4, 8, 16, 32, 64}) names.push_back(std::string("jl_moe_matvec_") + tag + "_l" + std::to_string(lpr));
    const int types[] = {JL_TYPE_Q4_K, JL_TYPE_Q8_0, JL_TYPE_Q6_K};
    for (int t : types)
        for (int rpw : {1, 2, 4}) {
            char nm[64];
            snprintf(nm, sizeof nm, "jl_matvec_%s_r%d", type_info(t)->tag, rpw);
            names.push_back(nm);
            names.push_back(std::string(nm) + "_x4");
        }
    for (int rpw : {1, 2, 4}) names.push_back("jl_matvec_q8_0p_r" + std::to_string(rpw) + "_x4");
    for (const char* tag : {"q4k", "q8_0", "q6k", "q8_0p"}) {
        names.push_back(std::string("jl_matvec_multi_") + tag);
        names.push_back(std::string("jl_matvec_multi_") + tag + "_x4");
        names.push_back(std::string("jl_matvec_multi_") + tag + "_q");
    }
    names.push_back("jl_matvec_segments");
    for (const char* tag : {"q4k", "q8_0", "q6k"})
        for (int rw : {16, 32, 64})
            for (const char* form : {"", "act_", "norm_"})
                names.push_back(std::string("jl_matvec_packed_multi_") + form + tag + "_w" + std::to_string(rw));
    for (const auto& n : names) {
        hipFunction_t f;
        e = H->ModuleGetFunction(&f, c->module, n.c_str());
        if (e != hipSuccess)
            return bail(JL_ERR_HIP, "hipModuleGetFunction(" + n + "): " + H->GetErrorString(e));
        c->fn[n] = f;
    }
    {
        uint32_t tab[2 * 17];
        for (uint32_t n = 0; n <= 16; n++) { tab[2 * n] = 0; tab[2 * n + 1] = n; }
        e = H->Malloc((void**)&c->one_group, sizeof tab);
        if (e == hipSuccess) e = H->Memcpy(c->one_group, tab, sizeof tab, hipMemcpyHostToDevice);
        if (e != hipSuccess) return bail(JL_ERR_HIP, std::string("column range table: ") + H->GetErrorString(e));
    }
    *out = c;
    return JL_OK;
}

const char* jl_hip_runtime(void) {
    std::string why;
    const HipApi* h = hip_api(&why);
    return h ? h->path.c_str() : "";
}

void jl_ctx_destroy(jl_ctx* c) {
    if (!c) return;
    if (c->no_device) {
        delete c;
        return;
    }
    (void)H->SetDevice(c->device);
    if (c->stream) (void)H->StreamSynchronize(c->stream);
    (void)H->DeviceSynchronize();   // callers' streams may still read the workspaces
    for (auto& kv : c->resident) (void)H->Free(kv.second.dev);
    if (c->gemm_ws) (void)H->Free(c->gemm_ws);
    if (c->w16_ws) (void)H->Free(c->w16_ws);
    if (c->moe_ws) (void)H->Free(c->moe_ws);
    if (c->unpack_ws) (void)H->Free(c->unpack_ws);
    if (c->flag_ws) (void)H->Free(c->flag_ws);
    if (c->moe_q_ws) (void)H->Free(c->moe_q_ws);
    if (c->act_ws) (void)H->Free(c->act_ws);
    if (c->layer_ws) (void)H->Free(c->layer_ws);
    if (c->moe_route_ws) (void)H->Free(c->moe_route_ws);
    for (auto& kv : c->layers)
        if (kv.second.mem) (void)H->Free(kv.second.mem);
    if (c->one_group) (void)H->Free(c->one_group);
    if (c->mx_ws) (void)H->Free(c->mx_ws);
    if (c->stage_x) (void)H->Free(c->stage_x);
    if (c->stage_out) (void)H->Free(c->stage_out);
    if (c->module) (void)H->ModuleUnload(c->module);
    if (c->stream) (void)H->StreamDestroy(c->stream);
    delete c;
}

const char* jl_last_error(const jl_ctx* c) { return c ? c->err.c_str() : g_create_error.c_str(); }

int jl_set_act_window(jl_ctx* c, int window) {
    if (!c) return JL_ERR_ARG;
    if (window != 32 && window != 64 && window != 128 && window != 256)
        return fail(c, JL_ERR_ARG, "act_window must be 32, 64, 128 or 256, not %d", window);
    c->act_window = window;
    return JL_OK;
}

void* jl_stream(jl_ctx* c) { return c ? (void*)c->stream : nullptr; }

int jl_synchronize(jl_ctx* c) {
    if (!c) return JL_ERR_ARG;
    HIP_TRY(c, H->SetDevice(c->device));
    HIP_TRY(c, H->StreamSynchronize(c->stream));
    return JL_OK;
}

unsigned long long jl_launch_count(const jl_ctx* c) { return c ? c->launches.load() : 0ull; }

int jl_set_tuning(jl_ctx* c, const char* key, int value) {
    if (!c || !key) return JL_ERR_ARG;
    if (!strcmp(key, "matvec.rpw")) c->tune.rpw = value;
    else if (!strcmp(key, "matvec.block")) c->tune.block = value;
    else if (!strcmp(key, "matvec.grid")) c->tune.grid = value;
    else if (!strcmp(key, "packed.rw")) c->tune.packed_rw = value;
    else if (!strcmp(key, "packed.block")) c->tune.packed_block = value;
    else if (!strcmp(key, "moe.group")) c->tune.moe_group = value;
    else if (!strcmp(key, "moe.logits")) c->tune.moe_logits = value;
    else if (!strcmp(key, "moe.q6k_cols")) c->tune.moe_q6k_cols = value;
    else if (!strcmp(key, "moe.shares")) c->tune.moe_shares = value;
    else if (!strcmp(key, "moe.form")) c->tune.moe_form = value;
    else if (!strcmp(key, "moe.group16")) c->tune.moe_g16 = value;
    else if (!strcmp(key, "moe.chunk")) c->tune.moe_chunk = value;
    else if (!strcmp(key, "moe.waves")) c->tune.moe_waves = value;
    else if (!strcmp(key, "moe.lpr")) c->tune.moe_lpr = value;
    else if (!strcmp(key, "gemm.rows")) c->tune.gemm_rows = value;
    else if (!strcmp(key, "mxfp4.split")) c->tune.mx_split = value;
    else if (!strcmp(key, "mxfp4.rows")) c->tune.mx_rows = value;
    else if (!strcmp(key, "mxfp4.planes")) c->tune.mx_planes = value;
    else if (!strcmp(key, "mxfp4.scaled")) c->tune.mx_scaled = value;
    else if (!strcmp(key, "matvec.q8pair")) c->tune.q8pair = value;
    else if (!strcmp(key, "matvec.xpre")) c->tune.xpre = value;
    else if (!strcmp(key, "matvec.act_split")) c->tune.act_split = value;
    else if (!strcmp(key, "gemm.form")) c->tune.gemm_form = value;
    else if (!strcmp(key, "gemm.fold")) c->tune.gemm_fold = value;
    else if (!strcmp(key, "gemm.fold_waves")) c->tune.gemm_fold_waves = value;
    else if (!strcmp(key, "gemm.split")) c->tune.gemm_split = value;
    else if (!strcmp(key, "gemm.prep")) c->tune.gemm_prep = value;
    else if (!strcmp(key, "gemm.planes")) c->tune.gemm_planes = value;
    else if (!strcmp(key, "gemm.min_tok")) c->gemm_min_tok = value > 0 ? value : 3;
    else return fail(c, JL_ERR_ARG, "unknown tuning key %s", key);
    return JL_OK;
}

/* ------------------------------------------------ device-pointer entry points */

int jl_quantize_act_dev(jl_ctx* c, const float* x, int ntok, int k, int8_t* q, float* as,
                        float* sum16, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!x || !q || !as || !sum16 || ntok <= 0 || k <= 0)
        return fail(c, JL_ERR_ARG, "quantize_act: bad operand");
    if (k % 32 != 0 || !aligned16(x) || !aligned16(q)) return JL_DECLINED;
    if (ntok > 65535) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    int per = c->act_window / 32;
    const float* no_gate = nullptr;
    void* params[] = {(void*)&x, (void*)&q, (void*)&as, (void*)&sum16, (void*)&k, (void*)&per, (void*)&no_gate};
    unsigned gx = (unsigned)((k / 4 + 255) / 256);  // one thread per four elements
    return launch(c, "jl_quantize_act", gx, (unsigned)ntok, 256, 0, pick_stream(c, stream), params);
}

int jl_dequant_dev(jl_ctx* c, int type, const void* src, float* dst, size_t n, void* stream) {
    if (!c) return JL_ERR_ARG;
    int be;
    switch (type) {
    case JL_TYPE_Q8_0: case JL_TYPE_MXFP4: be = 32; break;
    case JL_TYPE_Q4_K: case JL_TYPE_Q6_K: be = 256; break;
    default: return JL_DECLINED;
    }
    if (!src || !dst) return fail(c, JL_ERR_ARG, "dequant: null operand");
    if (n == 0 || n % (size_t)be != 0) return fail(c, JL_ERR_ARG, "dequant: %zu elements is not whole blocks", n);
    if (type == JL_TYPE_Q4_K && ((uintptr_t)src & 3) != 0) return JL_DECLINED;
    if (type != JL_TYPE_MXFP4 && ((uintptr_t)src & 1) != 0) return JL_DECLINED;
    size_t blocks = (n + 255) / 256;
    if (blocks > 0x7fffffffu) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    void* params[] = {(void*)&src, (void*)&dst, (void*)&n, (void*)&type};
    return launch(c, "jl_dequant", (unsigned)blocks, 1, 256, 0, pick_stream(c, stream), params);
}

int jl_matvec_dev(jl_ctx* c, float* out, int type, const void* w, const float* x, int nrows, int k,
                  void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!x) return fail(c, JL_ERR_ARG, "matvec: null x");
    HIP_TRY(c, H->SetDevice(c->device));
    return matvec_launch(c, out, type, w, x, nullptr, nullptr, nullptr, nrows, k, pick_stream(c, stream));
}

int jl_matvec_q8_dev(jl_ctx* c, float* out, int type, const void* w, const int8_t* q,
                     const float* as, const float* sum16, int nrows, int k, void* stream) {
    if (!c) return JL_ERR_ARG;
    HIP_TRY(c, H->SetDevice(c->device));
    return matvec_launch(c, out, type, w, nullptr, q, as, sum16, nrows, k, pick_stream(c, stream));
}

int jl_matvec_group_dev(jl_ctx* c, const jl_mv_group* g, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!g || g->n < 1 || g->n > JL_MAX_GROUP || !g->x || g->k <= 0) return fail(c, JL_ERR_ARG, "matvec group: bad group");
    HIP_TRY(c, H->SetDevice(c->device));
    hipStream_t st = pick_stream(c, stream);
    // everything is checked before the first launch: a group is served whole or not at all
    for (int i = 0; i < g->n; i++) {
        const TypeInfo* ti = nullptr;
        int rc = matvec_check(c, g->type[i], g->rows[i], g->k, &ti);
        if (rc != JL_OK) return rc;
        if (!g->out[i] || !g->w[i]) return fail(c, JL_ERR_ARG, "matvec group: null operand");
        if ((g->type[i] == JL_TYPE_Q4_K && !aligned16(g->w[i])) || ((uintptr_t)g->w[i] & 1)) return JL_DECLINED;
    }
    if (!aligned16(g->x) || (g->act_up && !aligned16(g->act_up))) return JL_DECLINED;
    if ((g->norm_w && !aligned16(g->norm_w)) || (g->norm_out && (!g->norm_w || !aligned16(g->norm_out)))) return JL_DECLINED;
    // one launch: the single-type kernel, or the mixed-type one when the formats differ
    // (the reference's MatVecSegments, jit/gpu/kernels/matvec.go:1411-1431)
    bool mixed = false;
    for (int i = 1; i < g->n; i++) mixed = mixed || g->type[i] != g->type[0];
    return matvec_multi_launch(c, g->type[0], g->n, g->out, g->w, g->rows, g->x, 0, g->act_up, g->resid, g->alpha,
                               g->k, st, g->norm_w, g->norm_eps, g->norm_out, mixed ? g->type : nullptr,
                               g->resid_gate);
}

int jl_matvec_packed_multi_dev(jl_ctx* c, float* const* outs, int type, const uint32_t* const* qs,
                               const uint32_t* const* d, const uint32_t* const* sc, const int* row0, int stride,
                               const float* x, size_t xstride, const float* up, float* resid, float alpha,
                               const float* resid_gate, const float* norm_w, float norm_eps, float* norm_out,
                               int nrows, int k, int m, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!outs || !qs || !d || !row0 || m < 1) return fail(c, JL_ERR_ARG, "packed multi: bad operand");
    if (m > JL_MAX_MULTI) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    PlaneRef pls[JL_MAX_MULTI];
    for (int j = 0; j < m; j++) {
        pls[j].qs = qs[j]; pls[j].d = d[j]; pls[j].sc = sc ? sc[j] : nullptr;
        pls[j].row = row0[j]; pls[j].stride = stride;
    }
    return packed_matvec_multi_launch(c, type, m, outs, pls, x, xstride, up, resid, alpha, resid_gate, norm_w,
                                      norm_eps, norm_out, nrows, k, pick_stream(c, stream));
}

int jl_matvec_multi_dev(jl_ctx* c, float* const* outs, int type, const void* const* ws, const float* x,
                        int nrows, int k, int m, void* stream) {
    return jl_matvec_gather_dev(c, outs, type, ws, x, 0, nullptr, nrows, k, m, stream);
}

int jl_matvec_gather_dev(jl_ctx* c, float* const* outs, int type, const void* const* ws, const float* x,
                         size_t xstride, const float* up, int nrows, int k, int m, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!outs || !ws || m < 1) return fail(c, JL_ERR_ARG, "matvec multi: bad operand");
    if (m > JL_MAX_MULTI) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    int rows[JL_MAX_MULTI];
    for (int i = 0; i < m; i++) rows[i] = nrows;
    return matvec_multi_launch(c, type, m, outs, ws, rows, x, xstride, up, nullptr, 0.f, k, pick_stream(c, stream));
}

int jl_matmul_dev(jl_ctx* c, float* out, int type, const void* w, const float* x, int nrows, int k,
                  int ntok, void* stream) {
    if (!c) return JL_ERR_ARG;
    HIP_TRY(c, H->SetDevice(c->device));
    return matmul_launch(c, out, type, w, x, nrows, k, ntok, pick_stream(c, stream));
}

int jl_matmul_static_dev(jl_ctx* c, float* out, int type, const void* w, const float* x, int nrows, int k,
                         int ntok, void* stream) {
    if (!c) return JL_ERR_ARG;
    HIP_TRY(c, H->SetDevice(c->device));
    if (!c->static_scratch) return fail(c, JL_ERR_HIP, "the static scratch is not available: %s", c->static_err.c_str());
    // The call runs jl_matmul_dev's own launch path with every context workspace set aside:
    // whatever the path asks for is carved, in order, from the static array (grow() above), and
    // a shape that needs more than the array holds is an error before anything is launched
    // that would use the missing piece.  No hipMalloc, no hipFree, no synchronisation.
    struct Saved { void** buf; size_t* have; void* b; size_t h; };
    Saved saved[] = {{&c->gemm_ws, &c->gemm_ws_bytes, nullptr, 0}, {&c->w16_ws, &c->w16_ws_bytes, nullptr, 0},
                     {&c->mx_ws, &c->mx_ws_bytes, nullptr, 0},     {&c->moe_q_ws, &c->moe_q_ws_bytes, nullptr, 0},
                     {&c->unpack_ws, &c->unpack_ws_bytes, nullptr, 0}};
    for (auto& s : saved) { s.b = *s.buf; s.h = *s.have; *s.buf = nullptr; *s.have = 0; }
    // a dry run first: the sizes are checked against the array before the first real launch
    int rc;
    {
        CallScope no_alloc(c, false, true);
        {
            CallScope dry(c, true, false);
            rc = matmul_launch(c, out, type, w, x, nrows, k, ntok, pick_stream(c, stream));
        }
        if (rc == JL_OK) {
            for (auto& s : saved) { *s.buf = nullptr; *s.have = 0; }
            g_call.static_used = 0;
            rc = matmul_launch(c, out, type, w, x, nrows, k, ntok, pick_stream(c, stream));
        }
    }
    for (auto& s : saved) { *s.buf = s.b; *s.have = s.h; }
    return rc;
}

size_t jl_static_scratch_bytes(void) { return JL_STATIC_SCRATCH_BYTES; }

int jl_packed_words(int type, int nrows, int k, size_t* nq, size_t* nd, size_t* nsc) {
    if (!nq || !nd || !nsc || nrows <= 0) return JL_ERR_ARG;
    return packed_words(type, (size_t)nrows, k, nq, nd, nsc) ? JL_OK : JL_DECLINED;
}

int jl_pack_weights_dev(jl_ctx* c, int type, const void* src, int nrows, int k, uint32_t* qs, uint32_t* d,
                        uint32_t* sc, void* stream) {
    if (!c) return JL_ERR_ARG;
    size_t nq, nd, nsc;
    if (nrows <= 0 || !packed_words(type, (size_t)nrows, k, &nq, &nd, &nsc)) return JL_DECLINED;
    if (!src || !qs || !d || (nsc && !sc)) return fail(c, JL_ERR_ARG, "pack: null operand");
    if (type != JL_TYPE_MXFP4 && ((uintptr_t)src & (type == JL_TYPE_Q4_K ? 3 : 1))) return JL_DECLINED;
    if (((uintptr_t)qs | (uintptr_t)d | (uintptr_t)sc) & 3) return JL_DECLINED;
    const int units = type == JL_TYPE_Q8_0 || type == JL_TYPE_MXFP4 ? k / 32 : k / 256;
    if (units > 65535) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    hipStream_t st = pick_stream(c, stream);
    PackArgs a;
    a.src = (const uint8_t*)src; a.qs = qs; a.d = d; a.sc = sc; a.nrows = nrows; a.k = k; a.type = type;
    a.flag = nullptr;
    void* params[] = {&a};
    if (type != JL_TYPE_MXFP4)
        return launch(c, "jl_pack_weights", (unsigned)((nrows + 255) / 256), (unsigned)units, 256, 0, st, params);
    // MXFP4: the packer raises a flag for a block whose exponent the D plane cannot hold
    // (mxfp4Refuse, jit/gpu/kernels/pack.go:407-420); the call waits for it, and a refused
    // matrix leaves the planes' contents undefined.
    int rc = ws_ensure(c, &c->flag_ws, &c->flag_ws_bytes, 256);
    if (rc != JL_OK) return rc;
    uint32_t flag = 0;
    HIP_TRY(c, H->Memcpy(c->flag_ws, &flag, 4, hipMemcpyHostToDevice));
    a.flag = (uint32_t*)c->flag_ws;
    rc = launch(c, "jl_pack_weights", (unsigned)((nrows + 255) / 256), (unsigned)units, 256, 0, st, params);
    if (rc != JL_OK) return rc;
    HIP_TRY(c, H->StreamSynchronize(st));
    HIP_TRY(c, H->Memcpy(&flag, c->flag_ws, 4, hipMemcpyDeviceToHost));
    return flag ? JL_DECLINED : JL_OK;
}

int jl_fold_admit_dev(jl_ctx* c, int type, const void* w, int nrows, int k, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (type != JL_TYPE_Q4_K || nrows <= 0 || k <= 0 || k % 256) return JL_DECLINED;
    if (!w) return fail(c, JL_ERR_ARG, "fold admit: null weights");
    if ((uintptr_t)w & 3) return JL_DECLINED;
    {
        std::lock_guard<std::mutex> g(c->forget_mu);
        c->fold_ok.erase((uintptr_t)w);   // whatever an earlier matrix at this address was found to be
    }
    HIP_TRY(c, H->SetDevice(c->device));
    hipStream_t st = pick_stream(c, stream);
    int rc = ws_ensure(c, &c->flag_ws, &c->flag_ws_bytes, 256);
    if (rc != JL_OK) return rc;
    uint32_t flag = 0;
    HIP_TRY(c, H->Memcpy(c->flag_ws, &flag, 4, hipMemcpyHostToDevice));
    FoldRangeArgs a;
    a.w = (const uint8_t*)w; a.nblocks = (size_t)nrows * (size_t)(k / 256); a.flag = (uint32_t*)c->flag_ws;
    void* params[] = {&a};
    rc = launch(c, "jl_q4k_fold_range", (unsigned)((a.nblocks + 255) / 256), 1, 256, 0, st, params);
    if (rc != JL_OK) return rc;
    HIP_TRY(c, H->StreamSynchronize(st));
    HIP_TRY(c, H->Memcpy(&flag, c->flag_ws, 4, hipMemcpyDeviceToHost));
    if (flag) return JL_DECLINED;
    std::lock_guard<std::mutex> g(c->forget_mu);
    c->fold_ok[(uintptr_t)w] = {nrows, k};
    return JL_OK;
}

int jl_unpack_weights_dev(jl_ctx* c, int type, const uint32_t* qs, const uint32_t* d, const uint32_t* sc,
                          int row, int stride, int nrows, int k, void* dst, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (type == JL_TYPE_MXFP4) {
        const PlaneRef mpl = {qs, d, nullptr, row, stride};
        int mrc = mx_planes_check(c, mpl, nrows, k);
        if (mrc != JL_OK) return mrc;
        if (!dst) return fail(c, JL_ERR_ARG, "unpack: null dst");
        HIP_TRY(c, H->SetDevice(c->device));
        return unpack_launch(c, type, mpl, nrows, k, dst, pick_stream(c, stream));
    }
    if (type != JL_TYPE_Q4_K && type != JL_TYPE_Q6_K && type != JL_TYPE_Q8_0) return JL_DECLINED;
    const PlaneRef pl = {qs, d, sc, row, stride};
    const TypeInfo* ti = nullptr;
    int rc = packed_check(c, type, pl, nrows, k, &ti);
    if (rc != JL_OK) return rc;
    if (!dst) return fail(c, JL_ERR_ARG, "unpack: null dst");
    if (((uintptr_t)dst & (type == JL_TYPE_Q4_K ? 3 : 1)) || k / ti->block_elems > 65535) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    return unpack_launch(c, type, pl, nrows, k, dst, pick_stream(c, stream));
}

int jl_matvec_packed_dev(jl_ctx* c, float* out, int type, const uint32_t* qs, const uint32_t* d,
                         const uint32_t* sc, int row, int stride, const float* x, int nrows, int k,
                         void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!x) return fail(c, JL_ERR_ARG, "packed matvec: null x");
    HIP_TRY(c, H->SetDevice(c->device));
    const PlaneRef pl = {qs, d, sc, row, stride};
    return packed_matvec_launch(c, out, type, pl, x, nullptr, nullptr, nullptr, nrows, k, pick_stream(c, stream));
}

int jl_matvec_packed_q8_dev(jl_ctx* c, float* out, int type, const uint32_t* qs, const uint32_t* d,
                            const uint32_t* sc, int row, int stride, const int8_t* q, const float* as,
                            const float* sum16, int nrows, int k, void* stream) {
    if (!c) return JL_ERR_ARG;
    HIP_TRY(c, H->SetDevice(c->device));
    const PlaneRef pl = {qs, d, sc, row, stride};
    return packed_matvec_launch(c, out, type, pl, nullptr, q, as, sum16, nrows, k, pick_stream(c, stream));
}

int jl_matmul_packed_dev(jl_ctx* c, float* out, int type, const uint32_t* qs, const uint32_t* d,
                         const uint32_t* sc, int row, int stride, const float* x, int nrows, int k,
                         int ntok, void* stream) {
    if (!c) return JL_ERR_ARG;
    HIP_TRY(c, H->SetDevice(c->device));
    const PlaneRef pl = {qs, d, sc, row, stride};
    return packed_matmul_launch(c, out, type, pl, x, nrows, k, ntok, pick_stream(c, stream));
}

int jl_reserve(jl_ctx* c, int max_tok, int max_k) {
    if (!c) return JL_ERR_ARG;
    if (max_tok <= 0 || max_k <= 0 || max_k % 256 != 0) return fail(c, JL_ERR_ARG, "reserve: %d x %d", max_tok, max_k);
    HIP_TRY(c, H->SetDevice(c->device));
    // the k-quant prep's layout and the window-32 prep's (fragments + two scale planes)
    const size_t tok_pad = ((size_t)max_tok + 255) / 256 * 256;
    const size_t w32 = (size_t)(max_k / 128) * (tok_pad / 32) * 8 * 1024 + 2 * (size_t)(max_k / 32) * tok_pad * 4;
    return gemm_ws_ensure(c, std::max(gemm_ws_need(max_tok, max_k), w32));
}

int jl_reserve_shape(jl_ctx* c, int type, int nrows, int k, int ntok, int packed) {
    if (!c) return JL_ERR_ARG;
    if (nrows <= 0 || k <= 0 || ntok <= 0) return fail(c, JL_ERR_ARG, "reserve shape: %d x %d, %d tokens", nrows, k, ntok);
    HIP_TRY(c, H->SetDevice(c->device));
    // Walk the call's own launch path with launching switched off: every workspace the path
    // would grow is grown now, by the code that sizes it for the real call.
    float* const out = (float*)(uintptr_t)4096;
    const float* const x = (const float*)(uintptr_t)4096;
    const void* const w = (const void*)(uintptr_t)4096;
    CallScope dry(c, true, false);
    int rc;
    if (type == JL_TYPE_MXFP4) {
        rc = packed ? jl_matmul_mxfp4_packed_bf16_dev(c, out, (const uint32_t*)w, (const uint32_t*)w, 0, nrows,
                                                      (const uint16_t*)w, nrows, k, ntok, nullptr)
                    : jl_matmul_mxfp4_bf16_dev(c, out, w, (const uint16_t*)w, nrows, k, ntok, nullptr);
    } else if (packed) {
        const PlaneRef pl = {(const uint32_t*)w, (const uint32_t*)w, (const uint32_t*)w, 0, nrows};
        rc = packed_matmul_launch(c, out, type, pl, x, nrows, k, ntok, c->stream);
    } else {
        rc = matmul_launch(c, out, type, w, x, nrows, k, ntok, c->stream);
    }
    return rc;
}

int jl_moe_route_dev(jl_ctx* c, const float* logits, int rows, int n_expert, int k_used, uint32_t* sel,
                     int sel_stride, float* wt, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!logits || !sel || !wt || rows <= 0 || n_expert <= 0 || k_used <= 0 || sel_stride < k_used)
        return fail(c, JL_ERR_ARG, "moe route: bad operand");
    if (n_expert > 1024 || k_used > 16 || k_used > n_expert) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    MoeRouteArgs a;
    a.logits = logits; a.sel = sel; a.wt = wt; a.n_expert = n_expert; a.k_used = k_used; a.sel_stride = sel_stride;
    void* params[] = {&a};
    // the form with the fewest experts a lane that holds them all (less code for a lone wavefront to fetch)
    const char* name = n_expert <= 128 ? "jl_moe_route_g2" : n_expert <= 256 ? "jl_moe_route_g4" : "jl_moe_route";
    return launch(c, name, (unsigned)rows, 1, 64, 0, pick_stream(c, stream), params);
}

int jl_moe_logits_dev(jl_ctx* c, float* logits, int wtype, const void* w, const float* x, int n_expert, int k,
                      int ntok, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!logits || !w || !x || n_expert <= 0 || k <= 0 || ntok <= 0)
        return fail(c, JL_ERR_ARG, "moe logits: bad operand");
    if (wtype != JL_TYPE_F32 && wtype != JL_TYPE_F16) return JL_DECLINED;
    if (((uintptr_t)w & (wtype == JL_TYPE_F32 ? 3 : 1)) || ((uintptr_t)x & 3)) return JL_DECLINED;
    if (n_expert > 65535 || (ntok + 7) / 8 > 65535) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    MoeLogitsArgs a;
    a.w = w; a.x = x; a.logits = logits; a.n_expert = n_expert; a.k = k; a.ntok = ntok;
    a.f16 = wtype == JL_TYPE_F16;
    void* params[] = {&a};
    // eight expert rows a workgroup once that still gives every CU three workgroups: 128
    // experts x k = 2048, 256 tokens 15.0 against 15.5 us, 2048 tokens 111 against 55
    // (tuning "moe.logits" = 1 / 8 forces a form)
    const long blocked = (long)((n_expert + 7) / 8) * ((ntok + 7) / 8);
    if (c->tune.moe_logits == 8 || (c->tune.moe_logits == 0 && blocked >= 3L * c->num_cu))
        return launch(c, "jl_moe_logits_e8", (unsigned)((n_expert + 7) / 8), (unsigned)((ntok + 7) / 8), 128, 0,
                      pick_stream(c, stream), params);
    return launch(c, "jl_moe_logits", (unsigned)n_expert, (unsigned)((ntok + 7) / 8), 128, 0,   // JL_LOGITS_TOK
                  pick_stream(c, stream), params);
}

int jl_moe_group_dev(jl_ctx* c, const uint32_t* sel, int sel_stride, int rows, int k_used, int n_expert,
                     uint32_t* start, uint32_t* perm, uint32_t* pos, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!sel || !start || !perm || !pos || rows <= 0 || k_used <= 0 || sel_stride < k_used)
        return fail(c, JL_ERR_ARG, "moe group: bad operand");
    if (n_expert <= 0 || n_expert > 1024) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    MoeGroupArgs a;
    a.sel = sel; a.start = start; a.perm = perm; a.pos = pos;
    a.sel_stride = sel_stride; a.rows = rows; a.k_used = k_used; a.n_expert = n_expert;
    void* params[] = {&a};
    // the linear-time form (moe.group = 1 forces the one that compares every pair with every
    // expert); a wavefront's share of the pairs is counted in 16 bits
    const size_t npairs = (size_t)rows * k_used;
    const size_t lds2 = 16 * (size_t)n_expert * 2 + ((size_t)n_expert + 17) * 4;   // JL_MOE_GROUP2_LDS
    // (an expert's running count, over all shares, is kept in 16 bits up to 65535 pairs and
    // in 32 bits above)
    if (c->tune.moe_group != 1 && lds2 <= c->lds_limit && npairs <= 65535)
        return launch(c, "jl_moe_group2", 1, 1, 1024, (unsigned)lds2, pick_stream(c, stream), params);
    const size_t lds2w = 16 * (size_t)n_expert * 4 + ((size_t)n_expert + 17) * 4;
    if (c->tune.moe_group != 1 && lds2w <= c->lds_limit && npairs <= 0x7fffffffu)
        return launch(c, "jl_moe_group2_wide", 1, 1, 1024, (unsigned)lds2w, pick_stream(c, stream), params);
    return launch(c, "jl_moe_group", 1, 1, 1024, 0, pick_stream(c, stream), params);
}

int jl_moe_matvec_dev(jl_ctx* c, float* out0, float* out1, int type, const void* bank0, const void* bank1,
                      const float* x, const float* x2, const uint32_t* src, const uint32_t* start,
                      int n_expert, int ncols, int nrows, int k, void* stream) {
    if (!c) return JL_ERR_ARG;
    HIP_TRY(c, H->SetDevice(c->device));
    return moe_matvec_launch(c, out0, out1, type, bank0, bank1, x, x2, src, start, n_expert, ncols, nrows, k,
                             pick_stream(c, stream));
}

int jl_moe_matvec_packed_dev(jl_ctx* c, float* out0, float* out1, int type, const jl_packed_bank* bank0,
                             const jl_packed_bank* bank1, const float* x, const float* x2, const uint32_t* src,
                             const uint32_t* start, int n_expert, int ncols, int nrows, int k, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!bank0) return fail(c, JL_ERR_ARG, "moe matvec: null bank");
    HIP_TRY(c, H->SetDevice(c->device));
    return moe_matvec_launch(c, out0, out1, type, nullptr, nullptr, x, x2, src, start, n_expert, ncols, nrows, k,
                             pick_stream(c, stream), bank0, bank1);
}

int jl_moe_combine_dev(jl_ctx* c, float* resid, const float* y, const float* wt, const uint32_t* sel,
                       int sel_stride, const uint32_t* pos, int rows, int k_used, int n_embd, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!resid || !y || !wt || !sel || !pos || rows <= 0 || n_embd <= 0)
        return fail(c, JL_ERR_ARG, "moe combine: bad operand");
    if (k_used <= 0 || k_used > 16 || sel_stride < k_used || rows > 65535) return JL_DECLINED;
    if (n_embd % 4 != 0 || !aligned16(resid) || !aligned16(y)) return JL_DECLINED;   // four columns a thread
    HIP_TRY(c, H->SetDevice(c->device));
    MoeCombineArgs a;
    a.resid = resid; a.y = y; a.wt = wt; a.sel = sel; a.pos = pos;
    a.sel_stride = sel_stride; a.k_used = k_used; a.n_embd = n_embd;
    void* params[] = {&a};
    return launch(c, "jl_moe_combine", (unsigned)((n_embd / 4 + 255) / 256), (unsigned)rows, 256, 0,
                  pick_stream(c, stream), params);
}

namespace {
// The routed block's workspace: first columns, row of a column, column of a pair, then gate, up
// and down of every column.
struct MoeWs {
    uint32_t *start, *perm, *pos;
    float *g, *u, *y;
};
int moe_ws(jl_ctx* c, int rows, int k_used, int n_expert, int n_ffn, int n_embd, MoeWs* w) {
    const size_t ncols = (size_t)rows * k_used;
    auto up256 = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t o_start = 0, o_perm = up256((size_t)(n_expert + 1) * 4), o_pos = o_perm + up256(ncols * 4);
    const size_t o_g = o_pos + up256(ncols * 4), o_u = o_g + up256(ncols * n_ffn * 4);
    const size_t o_y = o_u + up256(ncols * n_ffn * 4), total = o_y + up256(ncols * n_embd * 4);
    int rc = ws_ensure(c, &c->moe_ws, &c->moe_ws_bytes, total);
    if (rc != JL_OK) return rc;
    char* ws = (char*)c->moe_ws;
    w->start = (uint32_t*)(ws + o_start);
    w->perm = (uint32_t*)(ws + o_perm);
    w->pos = (uint32_t*)(ws + o_pos);
    w->g = (float*)(ws + o_g); w->u = (float*)(ws + o_u); w->y = (float*)(ws + o_y);
    return JL_OK;
}

int moe_ffn(jl_ctx* c, float* resid, int type, int down_type, const void* gate_bank, const void* up_bank,
            const void* down_bank, const jl_packed_bank* pg, const jl_packed_bank* pu, const jl_packed_bank* pd,
            const float* x, const uint32_t* sel, int sel_stride, const float* wt, int rows, int k_used, int n_expert,
            int n_ffn, int n_embd, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (rows <= 0 || k_used <= 0 || n_expert <= 0 || n_ffn <= 0 || n_embd <= 0)
        return fail(c, JL_ERR_ARG, "moe ffn: bad shape");
    if (n_expert > 1024 || k_used > 16 || n_ffn % 256 != 0 || n_embd % 256 != 0) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    hipStream_t st = pick_stream(c, stream);
    const size_t ncols = (size_t)rows * k_used;
    MoeWs w;
    int rc = moe_ws(c, rows, k_used, n_expert, n_ffn, n_embd, &w);
    if (rc != JL_OK) return rc;
    uint32_t *start = w.start, *perm = w.perm, *pos = w.pos;
    float *g = w.g, *u = w.u, *y = w.y;
    rc = jl_moe_group_dev(c, sel, sel_stride, rows, k_used, n_expert, start, perm, pos, st);
    if (rc != JL_OK) return rc;
    // gate and up: columns read the routed rows of x
    rc = moe_matvec_launch(c, g, u, type, gate_bank, up_bank, x, nullptr, perm, start, n_expert, (int)ncols, n_ffn, n_embd, st,
                           pg, pu);
    if (rc != JL_OK) return rc;
    // down: the activation of column c is silu(g[c]) * u[c]
    rc = moe_matvec_launch(c, y, nullptr, down_type, down_bank, nullptr, g, u, nullptr, start, n_expert, (int)ncols, n_embd, n_ffn, st,
                           pd, nullptr);
    if (rc != JL_OK) return rc;
    return jl_moe_combine_dev(c, resid, y, wt, sel, sel_stride, pos, rows, k_used, n_embd, st);
}

// The whole block from the hidden state on: router logits, softmax + top-k, the routed
// feed-forward.  (The three router steps as ONE launch -- the workgroup that stores a token
// group's last logit routes it, the one that routes the last group sorts the pairs -- measured
// slower than the launches it replaces, 117 us a 64-row block against 109: every hand-over inside
// a launch is a device-scope store, an atomic and a device-scope load one after the other, which
// costs what a launch boundary costs.)
int moe_block(jl_ctx* c, float* resid, int type, int down_type, const void* gate_bank, const void* up_bank,
              const void* down_bank, const jl_packed_bank* pg, const jl_packed_bank* pu, const jl_packed_bank* pd,
              int rtype, const void* router, const float* x, int rows, int k_used, int n_expert, int n_ffn, int n_embd,
              uint32_t* sel, float* wt, void* stream) {
    if (rows <= 0 || k_used <= 0 || n_expert <= 0 || n_ffn <= 0 || n_embd <= 0 || !router || !x || !resid)
        return fail(c, JL_ERR_ARG, "moe block: bad operand");
    if (n_expert > 1024 || k_used > 16 || k_used > n_expert || n_ffn % 256 != 0 || n_embd % 256 != 0) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    hipStream_t st = pick_stream(c, stream);
    const int sel_stride = k_used + 1;
    auto up256 = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t o_sel = up256((size_t)rows * n_expert * 4), o_wt = o_sel + up256((size_t)rows * sel_stride * 4);
    int rc = ws_ensure(c, &c->moe_route_ws, &c->moe_route_ws_bytes, o_wt + up256((size_t)rows * k_used * 4));
    if (rc != JL_OK) return rc;
    float* logits = (float*)c->moe_route_ws;
    if (!sel) sel = (uint32_t*)((char*)c->moe_route_ws + o_sel);
    if (!wt) wt = (float*)((char*)c->moe_route_ws + o_wt);
    rc = jl_moe_logits_dev(c, logits, rtype, router, x, n_expert, n_embd, rows, st);
    if (rc != JL_OK) return rc;
    rc = jl_moe_route_dev(c, logits, rows, n_expert, k_used, sel, sel_stride, wt, st);
    if (rc != JL_OK) return rc;
    return moe_ffn(c, resid, type, down_type, gate_bank, up_bank, down_bank, pg, pu, pd, x, sel, sel_stride, wt, rows, k_used,
                   n_expert, n_ffn, n_embd, st);
}
}  // namespace

int jl_moe_block_dev(jl_ctx* c, float* resid, int type, int down_type, const void* gate_bank, const void* up_bank,
                     const void* down_bank, int router_type, const void* router, const float* x, int rows, int k_used,
                     int n_expert, int n_ffn, int n_embd, uint32_t* sel, float* wt, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!gate_bank || !up_bank || !down_bank) return fail(c, JL_ERR_ARG, "moe block: null bank");
    return moe_block(c, resid, type, down_type, gate_bank, up_bank, down_bank, nullptr, nullptr, nullptr, router_type, router,
                     x, rows, k_used, n_expert, n_ffn, n_embd, sel, wt, stream);
}

int jl_moe_block_packed_dev(jl_ctx* c, float* resid, int type, const jl_packed_bank* gate, const jl_packed_bank* up,
                            const jl_packed_bank* down, int router_type, const void* router, const float* x, int rows,
                            int k_used, int n_expert, int n_ffn, int n_embd, uint32_t* sel, float* wt, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!gate || !up || !down) return fail(c, JL_ERR_ARG, "moe block: null bank");
    return moe_block(c, resid, type, type, nullptr, nullptr, nullptr, gate, up, down, router_type, router, x, rows, k_used,
                     n_expert, n_ffn, n_embd, sel, wt, stream);
}

int jl_moe_ffn_types_dev(jl_ctx* c, float* resid, int type, int down_type, const void* gate_bank, const void* up_bank,
                         const void* down_bank, const float* x, const uint32_t* sel, int sel_stride,
                         const float* wt, int rows, int k_used, int n_expert, int n_ffn, int n_embd, void* stream) {
    return moe_ffn(c, resid, type, down_type, gate_bank, up_bank, down_bank, nullptr, nullptr, nullptr, x, sel, sel_stride, wt,
                   rows, k_used, n_expert, n_ffn, n_embd, stream);
}

int jl_moe_ffn_packed_dev(jl_ctx* c, float* resid, int type, const jl_packed_bank* gate, const jl_packed_bank* up,
                          const jl_packed_bank* down, const float* x, const uint32_t* sel, int sel_stride,
                          const float* wt, int rows, int k_used, int n_expert, int n_ffn, int n_embd, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!gate || !up || !down) return fail(c, JL_ERR_ARG, "moe ffn: null bank");
    return moe_ffn(c, resid, type, type, nullptr, nullptr, nullptr, gate, up, down, x, sel, sel_stride, wt, rows, k_used,
                   n_expert, n_ffn, n_embd, stream);
}

int jl_moe_ffn_dev(jl_ctx* c, float* resid, int type, const void* gate_bank, const void* up_bank,
                   const void* down_bank, const float* x, const uint32_t* sel, int sel_stride,
                   const float* wt, int rows, int k_used, int n_expert, int n_ffn, int n_embd, void* stream) {
    return jl_moe_ffn_types_dev(c, resid, type, type, gate_bank, up_bank, down_bank, x, sel, sel_stride, wt, rows,
                                k_used, n_expert, n_ffn, n_embd, stream);
}

// ------------------------------------------------------------------ the block seam
namespace {
size_t up256(size_t v) { return (v + 255) & ~(size_t)255; }

// Bytes of one matrix (or bank of `sheets` sheets) of a plan: GGUF bytes, or its three planes
// (each rounded up to 256 bytes so that every plane starts aligned).
bool layer_matrix_bytes(int type, int packed, size_t nrows, int k, size_t* total, size_t plane[3]) {
    const TypeInfo* ti = type_info(type);
    if (!ti || k % ti->block_elems) return false;
    if (!packed) {
        *total = nrows * (size_t)(k / ti->block_elems) * ti->block_bytes;
        return true;
    }
    size_t nq, nd, nsc;
    if (nrows > 0x7fffffff || !packed_words(type, nrows, k, &nq, &nd, &nsc)) return false;
    plane[0] = nq * 4; plane[1] = nd * 4; plane[2] = nsc * 4;
    *total = up256(plane[0]) + up256(plane[1]) + up256(plane[2]);
    return true;
}
}  // namespace

int jl_prep_layer(jl_ctx* c, int li, const jl_layer_plan* plan) {
    if (!c) return JL_ERR_ARG;
    if (!plan || li < 0) return fail(c, JL_ERR_ARG, "prep layer: bad argument");
    const jl_layer_plan& P = *plan;
    if (P.n_embd <= 0 || P.n_ffn <= 0 || !P.gate || !P.up || !P.down)
        return fail(c, JL_ERR_ARG, "prep layer %d: missing weights or shape", li);
    const bool moe = P.kind == JL_LAYER_MOE;
    if (P.kind != JL_LAYER_DENSE && !moe) return fail(c, JL_ERR_ARG, "prep layer %d: kind %d", li, P.kind);
    if (moe && (P.n_expert < 1 || P.k_used < 1 || P.k_used > P.n_expert || !P.router))
        return fail(c, JL_ERR_ARG, "prep layer %d: mixture without router or experts", li);
    if (moe && (P.n_expert > 1024 || P.k_used > 16 || P.n_ffn % 256 || P.n_embd % 256)) return JL_DECLINED;
    if (moe && P.norm_w) return JL_DECLINED;
    if (P.packed && P.type != P.down_type && moe) return JL_DECLINED;   // packed banks: one type
    const size_t sheets = moe ? (size_t)P.n_expert : 1;
    size_t bg, bd, pg[3], pd[3];
    if (!layer_matrix_bytes(P.type, P.packed, sheets * P.n_ffn, P.n_embd, &bg, pg) ||
        !layer_matrix_bytes(P.down_type, P.packed, sheets * P.n_embd, P.n_ffn, &bd, pd))
        return JL_DECLINED;   // a type or shape without a kernel
    HIP_TRY(c, H->SetDevice(c->device));
    const size_t o_gate = 0, o_up = up256(bg), o_down = o_up + up256(bg), o_norm = o_down + up256(bd);
    const size_t o_router = o_norm + up256(P.norm_w ? (size_t)P.n_embd * 4 : 0);
    const size_t total = o_router + up256(moe ? (size_t)P.n_expert * P.n_embd * 4 : 0);
    jl_release_layers(c, li, li + 1);
    void* mem = nullptr;
    if (H->Malloc(&mem, total) != hipSuccess) {
        (void)H->GetLastError();
        return JL_DECLINED;   // the block does not fit: it stays on the host
    }
    Layer L;
    L.plan = P;
    L.plan.gate = L.plan.up = L.plan.down = nullptr;
    L.plan.norm_w = L.plan.router = nullptr;
    L.mem = mem;
    char* base = (char*)mem;
    auto fail_free = [&](hipError_t e, const char* what) {
        (void)H->Free(mem);
        return fail(c, JL_ERR_HIP, "prep layer %d: %s: %s", li, what, H->GetErrorString(e));
    };
    auto put = [&](size_t off, const void* src, size_t n) { return H->Memcpy(base + off, src, n, hipMemcpyHostToDevice); };
    hipError_t e = hipSuccess;
    if (!P.packed) {
        if ((e = put(o_gate, P.gate, bg)) != hipSuccess || (e = put(o_up, P.up, bg)) != hipSuccess ||
            (e = put(o_down, P.down, bd)) != hipSuccess)
            return fail_free(e, "weight upload");
        L.gate = base + o_gate; L.up = base + o_up; L.down = base + o_down;
    } else {
        auto put_planes = [&](size_t off, const void* hp, const size_t pl[3], const uint32_t* out[3]) {
            const jl_host_planes* h = (const jl_host_planes*)hp;
            const uint32_t* src[3] = {h->qs, h->d, h->sc};
            for (int i = 0; i < 3; i++) {
                out[i] = (const uint32_t*)(base + off);
                if (pl[i]) {
                    if (!src[i]) return hipErrorInvalidValue;
                    hipError_t ee = put(off, src[i], pl[i]);
                    if (ee != hipSuccess) return ee;
                }
                off += up256(pl[i]);
            }
            return hipSuccess;
        };
        if ((e = put_planes(o_gate, P.gate, pg, L.gp)) != hipSuccess || (e = put_planes(o_up, P.up, pg, L.upl)) != hipSuccess ||
            (e = put_planes(o_down, P.down, pd, L.dp)) != hipSuccess)
            return fail_free(e, "plane upload");
    }
    if (P.norm_w) {
        if ((e = put(o_norm, P.norm_w, (size_t)P.n_embd * 4)) != hipSuccess) return fail_free(e, "norm upload");
        L.norm_w = (const float*)(base + o_norm);
    }
    if (moe) {
        if ((e = put(o_router, P.router, (size_t)P.n_expert * P.n_embd * 4)) != hipSuccess) return fail_free(e, "router upload");
        L.router = (const float*)(base + o_router);
    }
    c->layers[li] = L;
    return JL_OK;
}

int jl_release_layers(jl_ctx* c, int lo, int hi) {
    if (!c) return JL_ERR_ARG;
    bool any = false;
    for (auto it = c->layers.lower_bound(lo); it != c->layers.end() && it->first < hi;) {
        if (!any && !c->no_device) {
            // kernels enqueued by earlier runs may still read the block
            (void)H->SetDevice(c->device);
            (void)H->DeviceSynchronize();
            any = true;
        }
        if (it->second.mem) (void)H->Free(it->second.mem);
        it = c->layers.erase(it);
    }
    return JL_OK;
}

int jl_layer_count(jl_ctx* c) { return c ? (int)c->layers.size() : 0; }

int jl_layer_ffn_dev(jl_ctx* c, int li, const float* h, float* resid, int n, void* stream) {
    if (!c) return JL_ERR_ARG;
    auto it = c->layers.find(li);
    if (it == c->layers.end()) return fail(c, JL_ERR_ARG, "layer %d is not prepared", li);
    if (!h || !resid || n <= 0) return fail(c, JL_ERR_ARG, "layer %d: bad operand", li);
    const Layer& L = it->second;
    const jl_layer_plan& P = L.plan;
    HIP_TRY(c, H->SetDevice(c->device));
    hipStream_t st = pick_stream(c, stream);
    const int E = P.n_embd, F = P.n_ffn;
    jl_packed_bank bg, bu, bd;
    if (P.packed) {
        const int sheets = P.kind == JL_LAYER_MOE ? P.n_expert : 1;
        bg = jl_packed_bank{L.gp[0], L.gp[1], L.gp[2], 0, sheets * F};
        bu = jl_packed_bank{L.upl[0], L.upl[1], L.upl[2], 0, sheets * F};
        bd = jl_packed_bank{L.dp[0], L.dp[1], L.dp[2], 0, sheets * E};
    }
    if (P.kind == JL_LAYER_MOE) {
        return moe_block(c, resid, P.type, P.down_type, L.gate, L.up, L.down, P.packed ? &bg : nullptr, P.packed ? &bu : nullptr,
                         P.packed ? &bd : nullptr, JL_TYPE_F32, L.router, h, n, P.k_used, P.n_expert, F, E, nullptr, nullptr, st);
    }
    // dense.  More than one row without a norm in front: the grouped kernels, the block as a
    // mixture of one expert that every row selects with weight 1.
    if (n > 1 && !L.norm_w && F % 256 == 0 && E % 256 == 0 && (!P.packed || P.type == P.down_type)) {
        const size_t o_wt = up256((size_t)n * 2 * 4);
        int rc = grow(c, &c->layer_ws, &c->layer_ws_bytes, o_wt + up256((size_t)n * 4));
        if (rc != JL_OK) return rc;
        uint32_t* sel = (uint32_t*)c->layer_ws;
        float* wt = (float*)((char*)c->layer_ws + o_wt);
        size_t n_sel = (size_t)n * 2, n_wt = (size_t)n;
        uint32_t zero = 0, one = 0x3F800000u;
        void* p0[] = {&sel, &n_sel, &zero};
        rc = launch(c, "jl_fill_u32", (unsigned)((n_sel + 255) / 256), 1, 256, 0, st, p0);
        if (rc != JL_OK) return rc;
        void* p1[] = {&wt, &n_wt, &one};
        rc = launch(c, "jl_fill_u32", (unsigned)((n_wt + 255) / 256), 1, 256, 0, st, p1);
        if (rc != JL_OK) return rc;
        rc = moe_ffn(c, resid, P.type, P.down_type, L.gate, L.up, L.down, P.packed ? &bg : nullptr, P.packed ? &bu : nullptr,
                     P.packed ? &bd : nullptr, h, sel, 2, wt, n, 1, 1, F, E, st);
        if (rc != JL_DECLINED) return rc;
    }
    // one row at a time: gate and up in one launch (the norm riding in front), down over
    // silu(gate) * up with the residual add riding on it
    const size_t fb = up256((size_t)F * 4);
    int rc = grow(c, &c->layer_ws, &c->layer_ws_bytes, 2 * fb + up256((size_t)E * 4));
    if (rc != JL_OK) return rc;
    float* g = (float*)c->layer_ws;
    float* u = (float*)((char*)c->layer_ws + fb);
    float* y = (float*)((char*)c->layer_ws + 2 * fb);   // down's own rows (resid takes them as they are made)
    for (int r = 0; r < n; r++) {
        const float* hr = h + (size_t)r * E;
        float* rr = resid + (size_t)r * E;
        float* gu[2] = {g, u};
        float* yo[1] = {y};
        if (!P.packed) {
            const void* wgu[2] = {L.gate, L.up};
            const int rgu[2] = {F, F};
            rc = matvec_multi_launch(c, P.type, 2, gu, wgu, rgu, hr, 0, nullptr, nullptr, 0.f, E, st, L.norm_w, P.norm_eps);
            if (rc != JL_OK) return rc;
            const void* wd[1] = {L.down};
            const int rd[1] = {E};
            rc = matvec_multi_launch(c, P.down_type, 1, yo, wd, rd, g, 0, u, rr, 1.0f, F, st);
        } else {
            PlaneRef pgu[2] = {{L.gp[0], L.gp[1], L.gp[2], 0, F}, {L.upl[0], L.upl[1], L.upl[2], 0, F}};
            rc = packed_matvec_multi_launch(c, P.type, 2, gu, pgu, hr, 0, nullptr, nullptr, 0.f, nullptr, L.norm_w,
                                            P.norm_eps, nullptr, F, E, st);
            if (rc != JL_OK) return rc;
            PlaneRef pd1[1] = {{L.dp[0], L.dp[1], L.dp[2], 0, E}};
            rc = packed_matvec_multi_launch(c, P.down_type, 1, yo, pd1, g, 0, u, rr, 1.0f, nullptr, nullptr, 0.f, nullptr,
                                            E, F, st);
        }
        if (rc != JL_OK) return rc;
    }
    return JL_OK;
}

int jl_matmul_mxfp4_bf16_dev(jl_ctx* c, float* out, const void* w, const uint16_t* x, int nrows, int k,
                             int ntok, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (!out || !w || !x || nrows <= 0 || k <= 0 || ntok <= 0)
        return fail(c, JL_ERR_ARG, "mxfp4 matmul: bad operand");
    if (k % 32 != 0 || k < 32 || !aligned16(x) || (k % 8) != 0) return JL_DECLINED;
    if ((size_t)(k / 32) * 17 > 0x7fffffffu || ntok > 65535 * 128) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    MxGemmArgs a;
    a.out = out; a.w = (const uint8_t*)w; a.x = x;
    a.nrows = nrows; a.k = k; a.ntok = ntok; a.row_bytes = (k / 32) * 17;
    a.nsplit = 1; a.part = nullptr; a.tok_pad = 0;
    void* params[] = {&a};
    hipStream_t st = pick_stream(c, stream);
    if (ntok == 1 && k <= 3 * 2048 && c->tune.mx_rows != 1) {
        // one token: the activation stays in registers while a wavefront walks its rows
        const int nbi = (k / 32 + 63) / 64;
        char name[32];
        snprintf(name, sizeof name, "jl_mxfp4_matvec1_b%d", nbi);
        // (a wavefront a workgroup: four wavefronts a workgroup of four rows each were 180 workgroups for
        // 2880 rows and left 76 CUs without one: 4.65 -> 4.18 us)
        return launch(c, name, (unsigned)((nrows + JL_MX1_RPW - 1) / JL_MX1_RPW), 1, 64, 0, st, params);
    }
    if (ntok <= 8)  // a handful of tokens: stream the rows once, no tile to fill
        return launch(c, "jl_mxfp4_matvec", (unsigned)((nrows + 3) / 4), 1, 256, 0, st, params);
    if (ntok <= 64 && c->tune.mx_rows != 96 && c->tune.mx_rows != 128) {
        // few tokens: 16-row workgroups whose wavefronts split K, one launch after a prep
        // that lays the activations out in the order the block decode produces
        const int nt = (ntok + 15) / 16, groups = (k + 127) / 128;
        int rc = gemm_ws_ensure(c, (size_t)groups * 4 * nt * 1024);
        if (rc != JL_OK) return rc;
        MxPrepArgs pa;
        pa.x = x; pa.xf = (uint16_t*)c->gemm_ws; pa.ntok = ntok; pa.tok_pad = 16 * nt; pa.k = k;
        void* pp[] = {&pa};
        rc = launch(c, "jl_mxfp4_prep_few", (unsigned)groups, (unsigned)nt, 256, 0, st, pp);
        if (rc != JL_OK) return rc;
        a.x = (const uint16_t*)c->gemm_ws; a.tok_pad = 16 * nt;
        char name[32];
        snprintf(name, sizeof name, "jl_mxfp4_few_t%d", nt);
        return launch(c, name, (unsigned)((nrows + 15) / 16), 1, 512, 0, st, params);
    }
    const unsigned lds = 2u * 128u * 264u * 2u;   // two weight stages [128][264] bf16
    if (lds > c->lds_limit) return JL_DECLINED;
    // activations into matrix-fragment order (tokens padded to whole tiles, K to whole stages)
    const int tok_pad = (ntok + 127) / 128 * 128, stages = (k + 255) / 256;
    int rc = gemm_ws_ensure(c, (size_t)stages * (tok_pad / 32) * 16 * 1024);
    if (rc != JL_OK) return rc;
    MxPrepArgs pa;
    pa.x = x; pa.xf = (uint16_t*)c->gemm_ws; pa.ntok = ntok; pa.tok_pad = tok_pad; pa.k = k;
    void* pp[] = {&pa};
    rc = launch(c, "jl_mxfp4_prep", (unsigned)stages, (unsigned)(tok_pad / 32), 256, 0, st, pp);
    if (rc != JL_OK) return rc;
    a.x = (const uint16_t*)c->gemm_ws; a.tok_pad = tok_pad;
    // A grid that leaves most CUs idle is widened along K: each split writes partial sums
    // to a workspace slab and a second kernel adds the slabs in order.
    // rows per tile: 128, or 96 where that takes fewer rounds x rows (2880 rows x 1024 tokens:
    // 184 tiles of 128 rows leave 72 CUs idle for a whole tile, 240 of 96 rows do not)
    auto cost = [&](int rows) {
        const long t = (long)(tok_pad / 128) * ((nrows + rows - 1) / rows);
        return ((t + c->num_cu - 1) / c->num_cu) * rows;
    };
    const int trows = c->tune.mx_rows == 96 || c->tune.mx_rows == 128 ? c->tune.mx_rows
                      : (cost(96) < cost(128) ? 96 : 128);
    const char* gemm_name = trows == 96 ? "jl_mxfp4_gemm_r96" : "jl_mxfp4_gemm";
    const int tiles = (tok_pad / 128) * ((nrows + trows - 1) / trows);
    int nsplit = c->tune.mx_split > 0 ? c->tune.mx_split : (tiles * 2 <= c->num_cu ? c->num_cu / tiles : 1);
    if (nsplit > 8) nsplit = 8;
    if (nsplit > stages) nsplit = stages;
    if (nsplit > 1) {
        const int per = (stages + nsplit - 1) / nsplit;
        nsplit = (stages + per - 1) / per;   // no empty split
    }
    if (nsplit > 1) {
        const size_t n = (size_t)ntok * nrows;
        rc = ws_ensure(c, &c->mx_ws, &c->mx_ws_bytes, n * nsplit * 4);
        if (rc != JL_OK) return rc;
        a.nsplit = nsplit; a.part = (float*)c->mx_ws;
        rc = launch(c, gemm_name, (unsigned)(tok_pad / 128), (unsigned)((nrows + trows - 1) / trows), 512, lds, st,
                    params, (unsigned)nsplit);
        if (rc != JL_OK) return rc;
        SumPartsArgs sa;
        sa.out = out; sa.part = a.part; sa.n = n; sa.nsplit = nsplit;
        void* sp[] = {&sa};
        return launch(c, "jl_sum_parts", (unsigned)((n + 255) / 256), 1, 256, 0, st, sp);
    }
    return launch(c, gemm_name, (unsigned)(tok_pad / 128), (unsigned)((nrows + trows - 1) / trows), 512,
                  lds, st, params);
}

int jl_matmul_mxfp4_packed_bf16_dev(jl_ctx* c, float* out, const uint32_t* qs, const uint32_t* d, int row,
                                    int stride, const uint16_t* x, int nrows, int k, int ntok, void* stream) {
    if (!c) return JL_ERR_ARG;
    const PlaneRef pl = {qs, d, nullptr, row, stride};
    int rc = mx_planes_check(c, pl, nrows, k);
    if (rc != JL_OK) return rc;
    if (!out || !x || ntok <= 0) return fail(c, JL_ERR_ARG, "mxfp4 packed matmul: bad operand");
    if (!aligned16(x)) return JL_DECLINED;
    HIP_TRY(c, H->SetDevice(c->device));
    hipStream_t st = pick_stream(c, stream);
    if (c->tune.mx_scaled == 1) {
        // opt-in: activations to MX fp8, the planes' codes and exponents straight into the
        // block-scaled matrix instruction (about three bits of every activation are lost)
        if (ntok > 65535 * 32 || k % 8 != 0) return JL_DECLINED;
        const int tok_pad = (ntok + 127) / 128 * 128, nks = (k + 63) / 64, ntt = tok_pad / 32;
        const size_t xa_bytes = (size_t)nks * ntt * 64 * 32;
        rc = gemm_ws_ensure(c, xa_bytes + (size_t)nks * ntt * 64);
        if (rc != JL_OK) return rc;
        MxScaledPrepArgs pa;
        pa.x = x; pa.xa = (uint32_t*)c->gemm_ws; pa.xs = (uint8_t*)c->gemm_ws + xa_bytes;
        pa.ntok = ntok; pa.tok_pad = tok_pad; pa.k = k;
        void* pp[] = {&pa};
        rc = launch(c, "jl_mxfp4_scaled_prep", (unsigned)((nks + 3) / 4), (unsigned)ntt, 256, 0, st, pp);
        if (rc != JL_OK) return rc;
        MxScaledGemmArgs ga;
        ga.out = out; ga.qs = qs; ga.d = d; ga.xa = pa.xa; ga.xs = pa.xs;
        ga.nrows = nrows; ga.k = k; ga.ntok = ntok; ga.tok_pad = tok_pad; ga.row0 = row; ga.stride = stride;
        void* gp[] = {&ga};
        if (65536u > c->lds_limit) return JL_DECLINED;
        const long stiles = (long)(tok_pad / 64) * ((nrows + 63) / 64);
        if (stiles > 0x7fffffffL / 2) return JL_DECLINED;
        return launch(c, "jl_mxfp4_scaled_gemm", (unsigned)(8 * ((stiles + 7) / 8)), 1, 256, 65536, st, gp);
    }
    if (ntok <= 8 && c->tune.mx_planes != 2) {
        // a handful of tokens: the planes are read where they lie, a lane a row
        MxPlanesArgs a;
        a.out = out; a.qs = qs; a.d = d; a.x = (const uint32_t*)x;
        a.nrows = nrows; a.k = k; a.ntok = ntok; a.row0 = row; a.stride = stride;
        a.nwaves = k / 32 < 16 ? k / 32 : 16;
        // rows a workgroup: 64 when that fills the CUs, else 32 or 16 (more, smaller workgroups)
        int rl = c->tune.mx_planes == 64 || c->tune.mx_planes == 32 || c->tune.mx_planes == 16 ? c->tune.mx_planes : 0;
        // (measured: 2880 rows 5.4 us at 16 against 6.8 at 64; 5760 rows 6.3 at 32 against 7.1 and 8.6)
        if (!rl) rl = (nrows + 63) / 64 * 10 >= c->num_cu * 7 ? 64 : ((nrows + 31) / 32 * 10 >= c->num_cu * 7 ? 32 : 16);
        char name[40];
        snprintf(name, sizeof name, "jl_mxfp4_matvec_planes_r%d", rl);
        void* params[] = {&a};
        return launch(c, name, (unsigned)((nrows + rl - 1) / rl), 1, (unsigned)(64 * a.nwaves),
                      (unsigned)(a.nwaves * 8 * 64 * 4), st, params);
    }
    // a grid of 64 x 64 tiles that gives most CUs a workgroup: the planes feed the matrix
    // instruction's weight operand as they lie (a plane word is a lane's eight K values)
    const long tiles = (long)((ntok + 63) / 64) * ((nrows + 63) / 64);
    if (c->tune.mx_planes != 2 && (c->tune.mx_planes == 3 || 2 * tiles >= c->num_cu) && ntok <= 65535 * 32 &&
        k % 8 == 0 && 65536u <= c->lds_limit) {
        const int tok_pad = (ntok + 63) / 64 * 64, nks = (k + 63) / 64, ntt = tok_pad / 32;
        rc = gemm_ws_ensure(c, (size_t)nks * ntt * 4 * 1024);
        if (rc != JL_OK) return rc;
        MxPlanesPrepArgs pa;
        pa.x = x; pa.xa = (uint32_t*)c->gemm_ws; pa.ntok = ntok; pa.tok_pad = tok_pad; pa.k = k;
        void* pp[] = {&pa};
        rc = launch(c, "jl_mxfp4_planes_prep", (unsigned)((nks + 3) / 4), (unsigned)ntt, 256, 0, st, pp);
        if (rc != JL_OK) return rc;
        MxPlanesGemmArgs ga;
        ga.out = out; ga.qs = qs; ga.d = d; ga.xa = pa.xa;
        ga.nrows = nrows; ga.k = k; ga.ntok = ntok; ga.tok_pad = tok_pad; ga.row0 = row; ga.stride = stride;
        void* gp[] = {&ga};
        if (tiles > 0x7fffffffL / 2) return JL_DECLINED;
        return launch(c, "jl_mxfp4_planes_gemm", (unsigned)(8 * ((tiles + 7) / 8)), 1, 256, 65536, st, gp);
    }
    // fewer tiles: the few-token and tiled forms stage GGUF blocks, so the rows are restored first
    rc = ws_ensure(c, &c->unpack_ws, &c->unpack_ws_bytes, (size_t)nrows * (size_t)(k / 32) * 17);
    if (rc != JL_OK) return rc;
    rc = unpack_launch(c, JL_TYPE_MXFP4, pl, nrows, k, c->unpack_ws, st);
    if (rc != JL_OK) return rc;
    return jl_matmul_mxfp4_bf16_dev(c, out, c->unpack_ws, x, nrows, k, ntok, st);
}

/* ------------------------------------------------------- host-pointer seam */

int jl_matvec(jl_ctx* c, float* out, int type, const void* w, size_t wbytes, const float* x,
              int nrows, int k) {
    return jl_matmul(c, out, type, w, wbytes, x, nrows, k, 1);
}

int jl_matmul(jl_ctx* c, float* out, int type, const void* w, size_t wbytes, const float* x,
              int nrows, int k, int ntok) {
    if (!c) return JL_ERR_ARG;
    CtxLock lock(c);
    drain_forget(c);
    if (c->no_device) return fail(c, JL_ERR_HIP, "this context is bound to no device");
    const TypeInfo* ti = nullptr;
    int rc = matvec_check(c, type, nrows, k, &ti);
    if (rc != JL_OK) return rc;
    if (!out || !w || !x || ntok <= 0) return fail(c, JL_ERR_ARG, "matmul: bad operand");
    size_t need = (size_t)nrows * (size_t)(k / ti->block_elems) * ti->block_bytes;
    if (wbytes < need)
        return fail(c, JL_ERR_ARG, "matmul: weight has %zu bytes, %dx%d needs %zu", wbytes, nrows, k, need);
    HIP_TRY(c, H->SetDevice(c->device));
    void* wd = nullptr;
    rc = resident_weight(c, w, need, &wd);
    if (rc != JL_OK) return rc;
    size_t xb = (size_t)ntok * k * 4, ob = (size_t)ntok * nrows * 4;
    if ((rc = ensure_stage(c, &c->stage_x, &c->stage_x_bytes, xb)) != JL_OK) return rc;
    if ((rc = ensure_stage(c, &c->stage_out, &c->stage_out_bytes, ob)) != JL_OK) return rc;
    HIP_TRY(c, H->MemcpyAsync(c->stage_x, x, xb, hipMemcpyHostToDevice, c->stream));
    rc = matmul_launch(c, (float*)c->stage_out, type, wd, (const float*)c->stage_x, nrows, k, ntok, c->stream);
    if (rc != JL_OK) {
        (void)H->StreamSynchronize(c->stream);
        return rc;
    }
    HIP_TRY(c, H->MemcpyAsync(out, c->stage_out, ob, hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(c, H->StreamSynchronize(c->stream));
    return JL_OK;
}

namespace {
// The three planes of a matrix in host memory as ONE device allocation keyed on the QS pointer
// (uploaded on first use, jl_forget over the QS pointer releases it).  Called with c->mu held.
int resident_planes(jl_ctx* c, int type, const PlaneRef& host, int k, PlaneRef* pl) {
    size_t nq, nd, nsc;
    if (!packed_words(type, (size_t)host.stride, k, &nq, &nd, &nsc)) return JL_DECLINED;
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t o_d = up(nq * 4), o_sc = o_d + up(nd * 4), total = o_sc + up(nsc * 4);
    void* dev = nullptr;
    auto it = c->resident.find(host.qs);
    if (it != c->resident.end() && it->second.bytes == total) {
        dev = it->second.dev;
    } else {
        if (it != c->resident.end()) {
            HIP_TRY(c, H->Free(it->second.dev));
            c->resident.erase(it);
        }
        HIP_TRY(c, H->Malloc(&dev, total));
        hipError_t e = H->Memcpy(dev, host.qs, nq * 4, hipMemcpyHostToDevice);
        if (e == hipSuccess) e = H->Memcpy((char*)dev + o_d, host.d, nd * 4, hipMemcpyHostToDevice);
        if (e == hipSuccess && nsc) e = H->Memcpy((char*)dev + o_sc, host.sc, nsc * 4, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            (void)H->Free(dev);
            return fail(c, JL_ERR_HIP, "plane upload: %s", H->GetErrorString(e));
        }
        c->resident[host.qs] = Resident{dev, total};
    }
    *pl = PlaneRef{(const uint32_t*)dev, (const uint32_t*)((char*)dev + o_d), (const uint32_t*)((char*)dev + o_sc),
                   host.row, host.stride};
    return JL_OK;
}

// Host floats -> the staging buffer at a float offset (the buffer is already large enough).
int stage_in(jl_ctx* c, size_t off, const float* src, size_t n) {
    HIP_TRY(c, H->MemcpyAsync((float*)c->stage_x + off, src, n * 4, hipMemcpyHostToDevice, c->stream));
    return JL_OK;
}
size_t up64(size_t n) { return (n + 63) & ~(size_t)63; }   // floats: keeps every staged vector 256-byte aligned
}  // namespace

int jl_matvec_packed(jl_ctx* c, float* out, int type, const uint32_t* qs, const uint32_t* d,
                     const uint32_t* sc, int row, int stride, const float* x, int nrows, int k) {
    return jl_matmul_packed(c, out, type, qs, d, sc, row, stride, x, nrows, k, 1);
}

int jl_matvec_packed_multi(jl_ctx* c, float* const* outs, int type, const uint32_t* const* qs,
                           const uint32_t* const* d, const uint32_t* const* sc, const int* row0, int stride,
                           const float* x, size_t xstride, const float* up, int act, int nrows, int k, int m) {
    if (!c) return JL_ERR_ARG;
    CtxLock lock(c);
    drain_forget(c);
    // one matrix is not a batch (packedmulti.go:31-33, 109): jl_matvec_packed serves it
    if (m < 2 || nrows <= 0 || k <= 0 || (xstride != 0 && xstride < (size_t)k)) return JL_DECLINED;
    if (up && act != JL_ACT_SILU) return JL_DECLINED;   // the one gated activation the kernels bake in
    if (!outs || !qs || !d || !row0 || !x) return fail(c, JL_ERR_ARG, "packed multi: null operand");
    if (up && xstride == 0) return fail(c, JL_ERR_ARG, "packed multi: a gated activation needs one activation a matrix");
    if (c->no_device) return fail(c, JL_ERR_HIP, "this context is bound to no device");
    const TypeInfo* ti = nullptr;
    for (int j = 0; j < m; j++) {
        if (!outs[j] || !qs[j] || !d[j]) return fail(c, JL_ERR_ARG, "packed multi: null operand of matrix %d", j);
        const PlaneRef host = {qs[j], d[j], sc ? sc[j] : nullptr, row0[j], stride};
        int rc = packed_check(c, type, host, nrows, k, &ti);
        if (rc != JL_OK) return rc;
    }
    HIP_TRY(c, H->SetDevice(c->device));
    std::vector<PlaneRef> pls((size_t)m);
    for (int j = 0; j < m; j++) {
        const PlaneRef host = {qs[j], d[j], sc ? sc[j] : nullptr, row0[j], stride};
        int rc = resident_planes(c, type, host, k, &pls[(size_t)j]);
        if (rc != JL_OK) return rc;
    }
    const size_t nx = xstride ? (size_t)(m - 1) * xstride + (size_t)k : (size_t)k, o_up = up64(nx);
    int rc = ensure_stage(c, &c->stage_x, &c->stage_x_bytes, (o_up + (up ? nx : 0)) * 4);
    if (rc != JL_OK) return rc;
    const size_t orow = up64((size_t)nrows);
    if ((rc = ensure_stage(c, &c->stage_out, &c->stage_out_bytes, (size_t)m * orow * 4)) != JL_OK) return rc;
    if ((rc = stage_in(c, 0, x, nx)) != JL_OK) return rc;
    if (up && (rc = stage_in(c, o_up, up, nx)) != JL_OK) return rc;
    const float* xd = (const float*)c->stage_x;
    const float* ud = up ? xd + o_up : nullptr;
    for (int j0 = 0; j0 < m; j0 += JL_MAX_MULTI) {   // sixteen matrices a launch
        const int n = std::min(m - j0, (int)JL_MAX_MULTI);
        float* od[JL_MAX_MULTI];
        for (int j = 0; j < n; j++) od[j] = (float*)c->stage_out + (size_t)(j0 + j) * orow;
        rc = packed_matvec_multi_launch(c, type, n, od, &pls[(size_t)j0], xd + (size_t)j0 * xstride, xstride,
                                        ud ? ud + (size_t)j0 * xstride : nullptr, nullptr, 0.f, nullptr, nullptr, 0.f,
                                        nullptr, nrows, k, c->stream);
        if (rc != JL_OK) {
            (void)H->StreamSynchronize(c->stream);
            return rc;
        }
    }
    for (int j = 0; j < m; j++)
        HIP_TRY(c, H->MemcpyAsync(outs[j], (float*)c->stage_out + (size_t)j * orow, (size_t)nrows * 4,
                                  hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(c, H->StreamSynchronize(c->stream));
    return JL_OK;
}

int jl_moe_grouped(jl_ctx* c, float* resid, int type, const void* gate_bank, const void* up_bank,
                   const void* down_bank, const float* x, const uint32_t* sel, int sel_stride, const float* wt,
                   int rows, int k_used, int n_expert, int n_ffn, int n_embd) {
    if (!c) return JL_ERR_ARG;
    CtxLock lock(c);
    drain_forget(c);
    if (rows <= 0 || k_used <= 0 || n_expert <= 0 || n_ffn <= 0 || n_embd <= 0 || sel_stride < k_used)
        return fail(c, JL_ERR_ARG, "moe grouped: bad shape");
    if (!resid || !gate_bank || !up_bank || !down_bank || !x || !sel || !wt)
        return fail(c, JL_ERR_ARG, "moe grouped: null operand");
    const TypeInfo* ti = type_info(type);
    if (!ti || n_embd % ti->block_elems || n_ffn % ti->block_elems) return JL_DECLINED;
    if (n_expert > 1024 || k_used > 16 || n_ffn % 256 != 0 || n_embd % 256 != 0) return JL_DECLINED;
    if (c->no_device) return fail(c, JL_ERR_HIP, "this context is bound to no device");
    HIP_TRY(c, H->SetDevice(c->device));
    // the three banks stay resident, each keyed on its host pointer
    const size_t bank = (size_t)n_expert * n_ffn * (size_t)(n_embd / ti->block_elems) * ti->block_bytes;
    void *gd = nullptr, *ud = nullptr, *dd = nullptr;
    int rc = resident_weight(c, gate_bank, bank, &gd);
    if (rc == JL_OK) rc = resident_weight(c, up_bank, bank, &ud);
    if (rc == JL_OK) rc = resident_weight(c, down_bank, bank, &dd);
    if (rc != JL_OK) return rc;
    // staged as floats: x, resid, wt, then the selections (32-bit words as well)
    const size_t nx = (size_t)rows * n_embd, o_res = up64(nx), o_wt = o_res + up64(nx),
                 o_sel = o_wt + up64((size_t)rows * k_used), total = o_sel + up64((size_t)rows * sel_stride);
    if ((rc = ensure_stage(c, &c->stage_x, &c->stage_x_bytes, total * 4)) != JL_OK) return rc;
    if ((rc = stage_in(c, 0, x, nx)) != JL_OK) return rc;
    if ((rc = stage_in(c, o_res, resid, nx)) != JL_OK) return rc;
    if ((rc = stage_in(c, o_wt, wt, (size_t)rows * k_used)) != JL_OK) return rc;
    if ((rc = stage_in(c, o_sel, (const float*)sel, (size_t)rows * sel_stride)) != JL_OK) return rc;
    float* base = (float*)c->stage_x;
    rc = moe_ffn(c, base + o_res, type, type, gd, ud, dd, nullptr, nullptr, nullptr, base, (const uint32_t*)(base + o_sel),
                 sel_stride, base + o_wt, rows, k_used, n_expert, n_ffn, n_embd, c->stream);
    if (rc != JL_OK) {
        (void)H->StreamSynchronize(c->stream);
        return rc;
    }
    HIP_TRY(c, H->MemcpyAsync(resid, base + o_res, nx * 4, hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(c, H->StreamSynchronize(c->stream));
    return JL_OK;
}

int jl_matvec_packed_group(jl_ctx* c, int n, float* const* outs, const int* types, const uint32_t* const* qs,
                           const uint32_t* const* d, const uint32_t* const* sc, const int* row, const int* stride,
                           const int* rows, const float* x, int k, const float* act_up, int act, float* resid,
                           float alpha) {
    if (!c) return JL_ERR_ARG;
    CtxLock lock(c);
    drain_forget(c);
    if (n < 1 || n > JL_MAX_GROUP || k <= 0) return JL_DECLINED;   // MaxGroup, packedgroup.go:12
    if (act_up && act != JL_ACT_SILU) return JL_DECLINED;
    if (!outs || !types || !qs || !d || !row || !stride || !rows || !x) return fail(c, JL_ERR_ARG, "packed group: null operand");
    if (c->no_device) return fail(c, JL_ERR_HIP, "this context is bound to no device");
    // nothing runs unless every matrix can (packedgroup.go:47-50)
    for (int i = 0; i < n; i++) {
        if (!outs[i] || !qs[i] || !d[i]) return fail(c, JL_ERR_ARG, "packed group: null operand of matrix %d", i);
        if (rows[i] <= 0) return JL_DECLINED;
        const TypeInfo* ti = nullptr;
        const PlaneRef host = {qs[i], d[i], sc ? sc[i] : nullptr, row[i], stride[i] ? stride[i] : rows[i]};
        int rc = packed_check(c, types[i], host, rows[i], k, &ti);
        if (rc != JL_OK) return rc;
    }
    HIP_TRY(c, H->SetDevice(c->device));
    PlaneRef pls[JL_MAX_GROUP];
    for (int i = 0; i < n; i++) {
        const PlaneRef host = {qs[i], d[i], sc ? sc[i] : nullptr, row[i], stride[i] ? stride[i] : rows[i]};
        int rc = resident_planes(c, types[i], host, k, &pls[i]);
        if (rc != JL_OK) return rc;
    }
    // staged: x, the gate's partner, the residual (matrix 0's rows)
    const size_t o_up = up64((size_t)k), o_res = o_up + (act_up ? up64((size_t)k) : 0);
    int rc = ensure_stage(c, &c->stage_x, &c->stage_x_bytes, (o_res + (resid ? up64((size_t)rows[0]) : 0)) * 4);
    if (rc != JL_OK) return rc;
    size_t o_out[JL_MAX_GROUP], total = 0;
    for (int i = 0; i < n; i++) { o_out[i] = total; total += up64((size_t)rows[i]); }
    if ((rc = ensure_stage(c, &c->stage_out, &c->stage_out_bytes, total * 4)) != JL_OK) return rc;
    if ((rc = stage_in(c, 0, x, (size_t)k)) != JL_OK) return rc;
    if (act_up && (rc = stage_in(c, o_up, act_up, (size_t)k)) != JL_OK) return rc;
    if (resid && (rc = stage_in(c, o_res, resid, (size_t)rows[0])) != JL_OK) return rc;
    const float* xd = (const float*)c->stage_x;
    const float* ud = act_up ? xd + o_up : nullptr;
    float* rd = resid ? (float*)c->stage_x + o_res : nullptr;
    // matrices of one type and row count that follow one another share a launch (a block's gate
    // and up); the residual rides on matrix 0 (MVGroup.Resid, packedgroup.go:32-36)
    for (int i = 0; i < n;) {
        int e = i + 1;
        while (e < n && types[e] == types[i] && rows[e] == rows[i] && pls[e].stride == pls[i].stride) e++;
        float* od[JL_MAX_GROUP];
        for (int j = i; j < e; j++) od[j - i] = (float*)c->stage_out + o_out[j];
        rc = packed_matvec_multi_launch(c, types[i], e - i, od, &pls[i], xd, 0, ud, i == 0 ? rd : nullptr, alpha, nullptr,
                                        nullptr, 0.f, nullptr, rows[i], k, c->stream);
        if (rc != JL_OK) {
            (void)H->StreamSynchronize(c->stream);
            return rc;
        }
        i = e;
    }
    for (int i = 0; i < n; i++)
        HIP_TRY(c, H->MemcpyAsync(outs[i], (float*)c->stage_out + o_out[i], (size_t)rows[i] * 4, hipMemcpyDeviceToHost,
                                  c->stream));
    if (resid) HIP_TRY(c, H->MemcpyAsync(resid, rd, (size_t)rows[0] * 4, hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(c, H->StreamSynchronize(c->stream));
    return JL_OK;
}

int jl_matmul_packed(jl_ctx* c, float* out, int type, const uint32_t* qs, const uint32_t* d,
                     const uint32_t* sc, int row, int stride, const float* x, int nrows, int k, int ntok) {
    if (!c) return JL_ERR_ARG;
    CtxLock lock(c);
    drain_forget(c);
    if (c->no_device) return fail(c, JL_ERR_HIP, "this context is bound to no device");
    const PlaneRef host = {qs, d, sc, row, stride};
    const TypeInfo* ti = nullptr;
    int rc = packed_check(c, type, host, nrows, k, &ti);
    if (rc != JL_OK) return rc;
    if (!out || !x || ntok <= 0) return fail(c, JL_ERR_ARG, "packed matmul: bad operand");
    HIP_TRY(c, H->SetDevice(c->device));
    PlaneRef pl;
    if ((rc = resident_planes(c, type, host, k, &pl)) != JL_OK) return rc;
    size_t xb = (size_t)ntok * k * 4, ob = (size_t)ntok * nrows * 4;
    if ((rc = ensure_stage(c, &c->stage_x, &c->stage_x_bytes, xb)) != JL_OK) return rc;
    if ((rc = ensure_stage(c, &c->stage_out, &c->stage_out_bytes, ob)) != JL_OK) return rc;
    HIP_TRY(c, H->MemcpyAsync(c->stage_x, x, xb, hipMemcpyHostToDevice, c->stream));
    rc = ntok == 1 ? packed_matvec_launch(c, (float*)c->stage_out, type, pl, (const float*)c->stage_x, nullptr,
                                          nullptr, nullptr, nrows, k, c->stream)
                   : packed_matmul_launch(c, (float*)c->stage_out, type, pl, (const float*)c->stage_x, nrows, k,
                                          ntok, c->stream);
    if (rc != JL_OK) {
        (void)H->StreamSynchronize(c->stream);
        return rc;
    }
    HIP_TRY(c, H->MemcpyAsync(out, c->stage_out, ob, hipMemcpyDeviceToHost, c->stream));
    HIP_TRY(c, H->StreamSynchronize(c->stream));
    return JL_OK;
}

int jl_forget(jl_ctx* c, const void* p, size_t n) {
    if (!c) return JL_ERR_ARG;
    if (!p || n == 0) return JL_OK;
    // Queue the range under a lock no launch or upload holds, so this returns from any thread --
    // also from inside a page-in that this context's own weight upload started.  Then, as the
    // reference does (jit/gpu/tier/forget.go:38-49), apply the queue at once if the context is
    // free: the device copies go now and a caller that never makes another host-pointer call
    // still gets its memory back.  A busy context (another thread's call, or this thread's own)
    // applies the queue at the start of its next host-pointer call; jl_ctx_destroy frees the rest.
    {
        std::lock_guard<std::mutex> g(c->forget_mu);
        c->pending_forget.emplace_back((uintptr_t)p, (uintptr_t)p + n);
        // a device range: the matrices admitted to the folded-scale form inside it
        c->fold_ok.erase(c->fold_ok.lower_bound((uintptr_t)p), c->fold_ok.lower_bound((uintptr_t)p + n));
    }
    if (c->mu_owner.load() != std::this_thread::get_id() && c->mu.try_lock()) {
        c->mu_owner.store(std::this_thread::get_id());
        drain_forget(c);
        c->mu_owner.store(std::thread::id());
        c->mu.unlock();
    }
    return JL_OK;
}

int jl_probe_dev(jl_ctx* c, int kind, const void* src, size_t nbytes, int grid, int block, void* stream) {
    if (!c) return JL_ERR_ARG;
    if (kind == 2) {
        // hold the stream: nbytes is microseconds here, at most a tenth of a second
        if (nbytes > 100000) return fail(c, JL_ERR_ARG, "probe: a wait of %zu us", nbytes);
        HIP_TRY(c, H->SetDevice(c->device));
        size_t ticks = nbytes * 100;   // the constant clock runs at 100 MHz
        void* none = nullptr;
        void* wp[] = {(void*)&none, (void*)&ticks, (void*)&none};
        return launch(c, "jl_probe_wait", 1, 1, 64, 0, pick_stream(c, stream), wp);
    }
    if (kind == 3 || kind == 4) {
        // matrix-core ceiling: nbytes is the rounds of four matrix instructions a wavefront issues
        if (nbytes == 0 || nbytes > 1000000) return fail(c, JL_ERR_ARG, "probe: %zu rounds", nbytes);
        if (grid <= 0) grid = c->num_cu;
        if (block <= 0) block = 512;
        if (block % 64 != 0 || block > 1024) return fail(c, JL_ERR_ARG, "probe: block=%d", block);
        HIP_TRY(c, H->SetDevice(c->device));
        void* none = nullptr;
        void* mp[] = {(void*)&none, (void*)&nbytes, (void*)&none};
        return launch(c, kind == 3 ? "jl_probe_mfma" : "jl_probe_mfma_v5", (unsigned)grid, 1, (unsigned)block, 0,
                      pick_stream(c, stream), mp);
    }
    if (kind != 0 && kind != 1) return fail(c, JL_ERR_ARG, "probe: kind %d", kind);
    if (grid <= 0) grid = 2 * c->num_cu;
    if (block <= 0) block = 1024;
    if (block % 64 != 0 || block > 1024) return fail(c, JL_ERR_ARG, "probe: block=%d", block);
    if (kind == 1 && (!src || ((uintptr_t)src & 1) != 0)) return fail(c, JL_ERR_ARG, "probe: src");
    HIP_TRY(c, H->SetDevice(c->device));
    size_t nvec = nbytes / 16;
    void* sink = nullptr;
    void* params[] = {(void*)&src, (void*)&nvec, (void*)&sink};
    return launch(c, kind ? "jl_probe_read" : "jl_probe_empty", (unsigned)grid, 1, (unsigned)block, 0,
                  pick_stream(c, stream), params);
}

int jl_ctx_lock(jl_ctx* c) {
    if (!c) return JL_ERR_ARG;
    c->mu.lock();
    c->mu_owner.store(std::this_thread::get_id());
    return JL_OK;
}

int jl_ctx_unlock(jl_ctx* c) {
    if (!c) return JL_ERR_ARG;
    c->mu_owner.store(std::thread::id());
    c->mu.unlock();
    return JL_OK;
}

size_t jl_resident_count(jl_ctx* c) {
    if (!c) return 0;
    CtxLock lock(c);
    drain_forget(c);
    return c->resident.size();
}

}  // extern "C"
