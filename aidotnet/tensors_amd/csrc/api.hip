// C ABI of libaidotnet_mi355.so (declared in include/aidotnet_mi355.h): argument validation,
// status codes, the per-context workspace, and nothing else.  Validation mirrors what the
// reference's managed backend checks before its native calls (non-positive dimensions,
// grouped-query ratio, head-dim limit: src/AiDotNet.Tensors/Engines/DirectGpu/HIP/
// HipBackend.HalfPrecision.cs:167-177, HipBackend.cs:6123-6141, GpuKernelGuards.cs:12-52).
#include "../../../include/aidotnet_mi355.h"
#include "launch.hpp"

#include <map>
#include <mutex>
#include <math.h>
#include <string>
#include <vector>
#include <cstdio>
#include <cstring>

namespace {

// Scratch memory of the allocation-free decode entry point (aidn_mi355_attn_decode_bf16_noalloc): the split-KV partials
// (m, l, acc[D]) per (batch, head, split).  One copy per device, held until the process ends; its device address is looked
// up once per device in aidn_mi355_create and only that address -- never the array's name -- is used by host code.
constexpr size_t kStaticScratchBytes = 8u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};      // device address of `scratch` on each device (null = not looked up yet)
std::mutex g_scratch_mu;

// Library-owned workspace of one stream.  Blocks are never freed before aidn_mi355_destroy: a kernel that is still queued,
// or a captured graph that holds the address, keeps a valid block when a later call needs a larger one.
struct WsSlot {
    void* cur = nullptr;
    size_t bytes = 0;
    std::vector<void*> retired;
};

struct Ctx {
    int device = 0;
    std::mutex mu;
    std::string last_error;
    std::map<void*, WsSlot> ws;  // keyed by stream: calls on different streams never share split partials or intermediates
    int force_tile = 0;
    int attn_fast_path = 1;      // 0: every attention shape takes the general kernel (parity tests hold the two against each other)
};

int fail(Ctx* c, int code, const char* what)
{
    if (c) {
        std::lock_guard<std::mutex> g(c->mu);
        c->last_error = what;
    }
    return code;
}

int hip_status(Ctx* c, hipError_t e, const char* where)
{
    if (e == hipSuccess) return AIDN_OK;
    char buf[256];
    snprintf(buf, sizeof buf, "%s: %s", where, hipGetErrorString(e));
    if (c) {
        std::lock_guard<std::mutex> g(c->mu);
        c->last_error = buf;
    }
    return (int)e;
}

// Workspace of `stream`, at least `bytes` large.  Growing allocates a new block and keeps the old one until destroy (no
// synchronisation, nothing queued or captured is invalidated).  While `stream` is being captured into a graph nothing may be
// allocated: the call fails with AIDN_ERR_WORKSPACE and the caller reserves beforehand (aidn_mi355_reserve_workspace, or one
// eager call of the same sequence).
int acquire_ws(Ctx* c, void* stream, size_t bytes, void** out)
{
    std::lock_guard<std::mutex> g(c->mu);
    WsSlot& slot = c->ws[stream];
    if (bytes > slot.bytes) {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing((hipStream_t)stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone) {
            c->last_error = "workspace: the stream is being captured and its workspace would have to grow; reserve it before the capture";
            return AIDN_ERR_WORKSPACE;
        }
        size_t want = bytes < (1u << 20) ? (1u << 20) : bytes;
        if (want < 2 * slot.bytes) want = 2 * slot.bytes;           // geometric growth bounds what the retired blocks hold
        want = (want + 255) & ~(size_t)255;
        void* p = nullptr;
        const hipError_t me = hipMalloc(&p, want);
        if (me != hipSuccess) {
            (void)hipGetLastError();
            // another stream of the process may be capturing in global mode: allocation is then refused although this stream is not
            // the one under capture -- the same situation for the caller as a capture of its own stream
            if (me == hipErrorStreamCaptureUnsupported || me == hipErrorStreamCaptureInvalidated || me == hipErrorStreamCaptureImplicit ||
                me == hipErrorStreamCaptureWrongThread) {
                c->last_error = "workspace: allocation refused while a stream capture is in progress; reserve the workspace before the capture";
                return AIDN_ERR_WORKSPACE;
            }
            c->last_error = "workspace: hipMalloc failed";
            return AIDN_ERR_OUT_OF_MEMORY;
        }
        if (slot.cur) slot.retired.push_back(slot.cur);
        slot.cur = p; slot.bytes = want;
    }
    *out = slot.cur;
    return AIDN_OK;
}

bool dense0(const int64_t* s) { return s[0] == 0 && s[1] == 0 && s[2] == 0; }

int fill_params(Ctx* c, const aidn_attn_desc* d, aidn::AttnParams& p)
{
    if (!d) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "attention: descriptor is null");
    if (d->B <= 0 || d->H <= 0 || d->Sq <= 0 || d->Sk <= 0 || d->D <= 0)
        return fail(c, AIDN_ERR_INVALID_ARGUMENT, "attention: dimensions must be positive");
    int hkv = d->Hkv > 0 ? d->Hkv : d->H;
    if (hkv > d->H || d->H % hkv != 0)
        return fail(c, AIDN_ERR_INVALID_ARGUMENT, "attention: H must be an integer multiple of Hkv");
    if (d->D > 256) return fail(c, AIDN_ERR_UNSUPPORTED, "attention: head dimension above 256");
    if (d->mask_mode < 0 || d->mask_mode > 2) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "attention: mask_mode must be 0, 1 or 2");
    p.B = d->B; p.H = d->H; p.Hkv = hkv; p.Sq = d->Sq; p.Sk = d->Sk; p.D = d->D;
    p.scale = d->scale; p.causal = d->causal != 0; p.qoff = d->causal_query_offset; p.softcap = d->softcap;
    p.mask_mode = d->mask_mode; p.out16 = d->out_is_16bit != 0; p.bias_bs = d->bias_batch_stride;
    auto set = [&](long long* dst, const int64_t* src, long long heads, long long rows) {
        if (dense0(src)) { dst[0] = heads * rows * d->D; dst[1] = rows * d->D; dst[2] = d->D; }
        else { dst[0] = src[0]; dst[1] = src[1]; dst[2] = src[2]; }
    };
    set(p.qs, d->q_strides, d->H, d->Sq);
    set(p.ks, d->k_strides, hkv, d->Sk);
    set(p.vs, d->v_strides, hkv, d->Sk);
    set(p.os, d->o_strides, d->H, d->Sq);
    return AIDN_OK;
}

int attn_common(void* ctx, void* stream, int kind, const aidn_attn_desc* d, const void* q, const void* k, const void* v,
                void* o, float* lse, const float* bias, const float* mask, float* weights)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!q || !k || !v || !o) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "attention: q, k, v and o must not be null");
    aidn::AttnParams p;
    int st = fill_params(c, d, p);
    if (st) return st;
    if (kind == 0 && p.out16) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "attention: fp32 kernel has no 16-bit output");
    if (p.mask_mode != 0 && !mask) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "attention: mask_mode set but mask is null");
    p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse; p.bias = bias; p.mask = p.mask_mode ? mask : nullptr; p.weights = weights;
    if (weights && !lse) {
        // the probabilities are rebuilt from the saved log-sum-exp: borrow the workspace for it
        size_t need = (size_t)p.B * p.H * p.Sq * sizeof(float);
        void* ws = nullptr;
        st = acquire_ws(c, stream, need, &ws);
        if (st) return st;
        p.lse = (float*)ws;
    }
    p.allow_fast_path = c->attn_fast_path;
    if (!(weights && !lse)) {
        // key-range partials of a call whose query tiles alone would leave most of the chip idle; a stream under capture whose
        // workspace would have to grow simply runs unsplit
        const size_t need = aidn::attn_fwd_workspace_bytes(kind, p);
        void* ws = nullptr;
        if (need && acquire_ws(c, stream, need, &ws) == AIDN_OK) { p.workspace = ws; p.workspace_bytes = need; }
    }
    return hip_status(c, aidn::attn_fwd((hipStream_t)stream, kind, p), "attn_fwd");
}

// scratch_override: non-null = split partials go there (capacity scratch_bytes) and nothing is allocated
int decode_common(void* ctx, void* stream, int kind, const aidn_attn_desc* d, const void* q, const void* k, const void* v,
                  void* o, float* lse, int splits, void* scratch_override = nullptr, size_t scratch_bytes = 0)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!q || !k || !v || !o) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "decode: q, k, v and o must not be null");
    aidn::AttnParams p;
    int st = fill_params(c, d, p);
    if (st) return st;
    if (p.Sq != 1) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "decode: Sq must be 1");
    if (kind == 0 && p.out16) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "decode: fp32 kernel has no 16-bit output");
    if (p.softcap > 0.0f || p.mask_mode != 0)
        return fail(c, AIDN_ERR_UNSUPPORTED, "decode: soft-cap and masks are not available here; use aidn_mi355_attn_fwd_* with Sq = 1");
    p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse; p.bias = nullptr; p.mask = nullptr; p.weights = nullptr;
    p.allow_fast_path = c->attn_fast_path;
    int eff = aidn::attn_decode_splits(kind, p, splits);
    size_t need = aidn::attn_decode_workspace_bytes(p, eff);
    void* ws = nullptr;
    if (scratch_override) {
        if (need > scratch_bytes)
            return fail(c, AIDN_ERR_UNSUPPORTED, "decode (allocation-free): batch x heads x splits x head dimension exceeds the static scratch buffer");
        ws = scratch_override;
    } else if (need) {
        st = acquire_ws(c, stream, need, &ws);
        if (st) return st;
    }
    return hip_status(c, aidn::attn_decode((hipStream_t)stream, kind, p, eff, ws), "attn_decode");
}

bool valid_activation(int act) { return act >= 0 && act <= 6; }

int gemm16_common(void* ctx, void* stream, int kind, const uint16_t* A, const uint16_t* B, void* C, int out32, int M, int N, int K,
                  const float* bias = nullptr, int act = 0, float act_param = 0.0f)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!A || !B || !C) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm: A, B and C must not be null");
    if (M <= 0 || N <= 0 || K <= 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm: dimensions must be positive");
    void* ws = nullptr;
    size_t need = c->force_tile == 0 ? aidn::gemm_16_workspace_bytes(M, N, K) : 0;
    if (need) {
        int st = acquire_ws(c, stream, need, &ws);
        if (st == AIDN_ERR_WORKSPACE) ws = nullptr;      // under capture and not reserved: the tiled kernel needs no workspace
        else if (st) return st;
    }
    if (!valid_activation(act)) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm: unknown activation");
    return hip_status(c, aidn::gemm_16((hipStream_t)stream, kind, A, B, C, out32, M, N, K, c->force_tile, ws, ws ? need : 0, bias, act, act_param),
                      "gemm_16");
}

int gemm16_rope_common(void* ctx, void* stream, int kind, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K,
                       const float* cosc, const float* sinc, int head_dim, int rope_cols, int seq_len, int start_position)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!A || !B || !C || !cosc || !sinc) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm_rope: buffers must not be null");
    if (M <= 0 || N <= 0 || K <= 0 || head_dim <= 0 || seq_len <= 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm_rope: dimensions must be positive");
    if (head_dim & 1) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm_rope: head dimension must be even");
    if (rope_cols < 0 || rope_cols > N || rope_cols % head_dim != 0 || (N & 1))
        return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm_rope: rope_cols must be a multiple of head_dim within N, and N even");
    if (start_position < 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm_rope: start position must not be negative");
    void* ws = nullptr;
    size_t need = c->force_tile == 0 ? aidn::gemm_16_workspace_bytes(M, N, K) : 0;
    if (need) {
        int st = acquire_ws(c, stream, need, &ws);
        if (st == AIDN_ERR_WORKSPACE) ws = nullptr;      // under capture and not reserved: the tiled kernel and a second launch for the rotation
        else if (st) return st;
    }
    const aidn::RopeEpilogue rope{cosc, sinc, head_dim, rope_cols, seq_len, start_position};
    return hip_status(c, aidn::gemm_16_rope((hipStream_t)stream, kind, A, B, C, M, N, K, c->force_tile, ws, ws ? need : 0, rope), "gemm_16_rope");
}

// [Wq|Wk|Wv] side by side in one [dModel, 3 dModel] matrix (three strided device copies), the weight operand of the fused
// QKV projection.
hipError_t gather_qkv(hipStream_t sm, const void* wq, const void* wk, const void* wv, void* packed, int dModel, size_t es)
{
    const void* w3[3] = {wq, wk, wv};
    for (int j = 0; j < 3; j++) {
        hipError_t e = hipMemcpy2DAsync((unsigned char*)packed + (size_t)j * dModel * es, (size_t)3 * dModel * es, w3[j], (size_t)dModel * es,
                                        (size_t)dModel * es, (size_t)dModel, hipMemcpyDeviceToDevice, sm);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// Multi-head attention forward as three launches and no permutes: fused [Wq|Wk|Wv] projection into a packed
// [B*S, 3*dModel] activation, attention reading it through strides and writing [B, S, H, d], output projection.
// kind: 0 fp32, 1 fp16, 2 bf16 (16-bit: every intermediate stays in the input type, accumulation in fp32).
// wqkv non-null: the caller's pre-packed [dModel, 3 dModel] weight (nothing is gathered); else wq, wk, wv are gathered into the
// workspace on every call.
int mha_common(void* ctx, void* stream, int kind, const void* input, const void* wq, const void* wk, const void* wv, const void* wqkv,
               const void* wo, const float* mask, int mask_mode, void* output, int B, int S, int dModel, int heads)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!input || !wo || !output || (!wqkv && (!wq || !wk || !wv)))
        return fail(c, AIDN_ERR_INVALID_ARGUMENT, "mha: input, weights and output must not be null");
    if (B <= 0 || S <= 0 || dModel <= 0 || heads <= 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "mha: dimensions must be positive");
    if (dModel % heads != 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "mha: dModel must be divisible by the number of heads");
    const int dHead = dModel / heads;
    if (dHead > 256) return fail(c, AIDN_ERR_UNSUPPORTED, "mha: head dimension above 256");
    if (mask_mode < 0 || mask_mode > 2) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "mha: mask_mode must be 0, 1 or 2");
    if (mask_mode != 0 && !mask) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "mha: mask_mode set but mask is null");
    const long long rows = (long long)B * S;
    if (rows > 0x7FFFFFFFLL || 3LL * dModel > 0x7FFFFFFFLL) return fail(c, AIDN_ERR_UNSUPPORTED, "mha: B*S or 3*dModel exceeds 2^31");
    const size_t es = kind == 0 ? 4 : 2;
    auto up = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const size_t wf_bytes = wqkv ? 0 : up((size_t)dModel * 3 * dModel * es), qkv_bytes = up((size_t)rows * 3 * dModel * es);
    const size_t cc_bytes = up((size_t)rows * dModel * es);
    void* ws = nullptr;
    int st = acquire_ws(c, stream, wf_bytes + qkv_bytes + cc_bytes, &ws);
    if (st) return st;
    unsigned char* wf = (unsigned char*)ws;
    unsigned char* qkv = wf + wf_bytes;
    unsigned char* cc = qkv + qkv_bytes;
    hipStream_t sm = (hipStream_t)stream;
    hipError_t e;
    if (!wqkv) {
        e = gather_qkv(sm, wq, wk, wv, wf, dModel, es);
        if (e != hipSuccess) return hip_status(c, e, "mha: weight gather");
    }
    const void* w3 = wqkv ? wqkv : (const void*)wf;
    const int M = (int)rows, N3 = 3 * dModel;
    const int tile32 = c->force_tile;
    if (kind == 0) e = aidn::gemm_f32(sm, (const float*)input, (const float*)w3, (float*)qkv, M, N3, dModel, 1.0f, 0.0f, 0, 1, 0, 0, 0, tile32);
    else e = aidn::gemm_16(sm, kind - 1, (const uint16_t*)input, (const uint16_t*)w3, qkv, 0, M, N3, dModel, c->force_tile, nullptr, 0);
    if (e != hipSuccess) return hip_status(c, e, "mha: QKV projection");

    aidn::AttnParams p{};
    p.q = qkv; p.k = qkv + (size_t)dModel * es; p.v = qkv + (size_t)2 * dModel * es; p.o = cc;
    p.lse = nullptr; p.bias = nullptr; p.mask = mask_mode ? mask : nullptr; p.weights = nullptr;
    p.B = B; p.H = heads; p.Hkv = heads; p.Sq = S; p.Sk = S; p.D = dHead;
    p.scale = 1.0f / sqrtf((float)dHead); p.causal = 0; p.qoff = 0; p.softcap = 0.0f; p.mask_mode = mask_mode; p.out16 = kind != 0;
    p.bias_bs = 0;
    p.allow_fast_path = c->attn_fast_path;
    for (int i = 0; i < 3; i++) { long long v = i == 0 ? (long long)S * N3 : (i == 1 ? dHead : N3); p.qs[i] = v; p.ks[i] = v; p.vs[i] = v; }
    p.os[0] = (long long)S * dModel; p.os[1] = dHead; p.os[2] = dModel;
    e = aidn::attn_fwd(sm, kind, p);
    if (e != hipSuccess) return hip_status(c, e, "mha: attention");

    if (kind == 0) e = aidn::gemm_f32(sm, (const float*)cc, (const float*)wo, (float*)output, M, dModel, dModel, 1.0f, 0.0f, 0, 1, 0, 0, 0, tile32);
    else e = aidn::gemm_16(sm, kind - 1, (const uint16_t*)cc, (const uint16_t*)wo, output, 0, M, dModel, dModel, c->force_tile, nullptr, 0);
    return hip_status(c, e, "mha: output projection");
}

// Attention over a paged K/V cache: pools [numBlocks, blockSize, kvHeads, headDim], logical key j in pool row
// blockTable[j / blockSize] * blockSize + j % blockSize.  numQueries == 1: decode kernel; otherwise causal prefill
// (query i at logical position startPos + i sees keys 0 .. startPos + i).
int paged_common(void* ctx, void* stream, int kind, const void* q, const void* kcache, const void* vcache, const int32_t* block_table,
                 void* o, int heads, int kv_heads, int head_dim, int block_size, int num_queries, int key_len, int start_pos,
                 float scale, int splits, bool decode)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!q || !kcache || !vcache || !block_table || !o)
        return fail(c, AIDN_ERR_INVALID_ARGUMENT, "paged attention: q, pools, block table and o must not be null");
    if (heads <= 0 || head_dim <= 0 || block_size <= 0 || num_queries <= 0 || key_len <= 0)
        return fail(c, AIDN_ERR_INVALID_ARGUMENT, "paged attention: heads, headDim, blockSize and lengths must be positive");
    if (head_dim > 256) return fail(c, AIDN_ERR_UNSUPPORTED, "paged attention: head dimension above 256");
    if (kv_heads <= 0) kv_heads = heads;
    if (kv_heads > heads || heads % kv_heads != 0)
        return fail(c, AIDN_ERR_INVALID_ARGUMENT, "paged attention: heads must be an integer multiple of kvHeads");
    if (start_pos < 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "paged attention: startPos must not be negative");
    aidn::AttnParams p{};
    p.q = q; p.k = kcache; p.v = vcache; p.o = o;
    p.B = 1; p.H = heads; p.Hkv = kv_heads; p.Sq = num_queries; p.Sk = key_len; p.D = head_dim;
    p.scale = scale; p.causal = decode ? 0 : 1; p.qoff = start_pos; p.softcap = 0.0f; p.mask_mode = 0; p.out16 = 0; p.bias_bs = 0;
    // q and o are [numQueries, heads, headDim]; pool rows are [kvHeads, headDim] wide
    p.qs[0] = 0; p.qs[1] = head_dim; p.qs[2] = (long long)heads * head_dim;
    p.os[0] = 0; p.os[1] = head_dim; p.os[2] = (long long)heads * head_dim;
    p.ks[0] = 0; p.ks[1] = head_dim; p.ks[2] = (long long)kv_heads * head_dim;
    p.vs[0] = 0; p.vs[1] = head_dim; p.vs[2] = (long long)kv_heads * head_dim;
    p.block_table = block_table; p.block_size = block_size; p.block_table_stride = 0;
    p.allow_fast_path = c->attn_fast_path;
    if (decode) {
        int eff = aidn::attn_decode_splits(kind, p, splits);
        size_t need = aidn::attn_decode_workspace_bytes(p, eff);
        void* ws = nullptr;
        if (need) { int st = acquire_ws(c, stream, need, &ws); if (st) return st; }
        return hip_status(c, aidn::attn_decode((hipStream_t)stream, kind, p, eff, ws), "paged attn_decode");
    }
    return hip_status(c, aidn::attn_fwd((hipStream_t)stream, kind, p), "paged attn_fwd");
}

int rope_common(void* ctx, void* stream, int kind, const void* in, const float* cosc, const float* sinc, void* out,
                int64_t rows, int head_dim, int seq_len, int start_position)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!in || !cosc || !sinc || !out) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "rope: buffers must not be null");
    if (rows <= 0 || head_dim <= 0 || seq_len <= 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "rope: dimensions must be positive");
    if (head_dim & 1) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "rope: head dimension must be even");
    if (start_position < 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "rope: start position must not be negative");
    return hip_status(c, aidn::rope_interleaved((hipStream_t)stream, kind, in, cosc, sinc, out, rows, head_dim, seq_len, start_position), "rope");
}

int convert_common(void* ctx, void* stream, int kind, const void* in, void* out, int64_t n)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (n < 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "convert: negative element count");
    if (n == 0) return AIDN_OK;
    if (!in || !out) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "convert: in and out must not be null");
    return hip_status(c, aidn::convert((hipStream_t)stream, kind, in, out, n), "convert");
}

}  // namespace

extern "C" {

AIDN_API int aidn_mi355_create(int device, void** ctx)
{
    if (!ctx) return AIDN_ERR_INVALID_ARGUMENT;
    *ctx = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0 || device < 0 || device >= count) return AIDN_ERR_NO_DEVICE;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) return AIDN_ERR_NO_DEVICE;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return AIDN_ERR_NO_DEVICE;   // the code object holds gfx950 ISA only
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return (int)e;
    if (device < kMaxDevices) {
        // device address of this device's copy of the static scratch array, looked up once with the device current
        std::lock_guard<std::mutex> g(g_scratch_mu);
        if (!g_scratch_ptr[device]) {
            void* ptr = nullptr;
            e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
            if (e != hipSuccess) return (int)e;
            g_scratch_ptr[device] = ptr;
        }
    }
    Ctx* c = new Ctx();
    c->device = device;
    *ctx = c;
    return AIDN_OK;
}

AIDN_API int aidn_mi355_destroy(void* ctx)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_OK;
    bool any = false;
    for (auto& kv : c->ws) any = any || kv.second.cur;
    if (any) {
        (void)hipSetDevice(c->device);
        (void)hipDeviceSynchronize();
        for (auto& kv : c->ws) {
            if (kv.second.cur) (void)hipFree(kv.second.cur);
            for (void* r : kv.second.retired) (void)hipFree(r);
        }
    }
    delete c;
    return AIDN_OK;
}

AIDN_API const char* aidn_mi355_last_error(void* ctx)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return "";
    std::lock_guard<std::mutex> g(c->mu);
    static thread_local std::string copy;
    copy = c->last_error;
    return copy.c_str();
}

AIDN_API const char* aidn_mi355_version(void) { return "aidotnet-mi355 0.1 (gfx950)"; }

AIDN_API int aidn_mi355_sync(void* ctx, void* stream)
{
    return hip_status((Ctx*)ctx, hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
}

AIDN_API int aidn_mi355_set_gemm_tile(void* ctx, int tile)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (tile != 0 && tile != 64 && tile != 65 && tile != 128 && tile != 129 && tile != 130 && tile != 131 && tile != 192 && tile != 193 && tile != 256)
        return fail(c, AIDN_ERR_INVALID_ARGUMENT, "tile must be 0, 64, 65 (64, direct-to-LDS kernel), 128, 129 (128, direct-to-LDS kernel), "
                                                  "130 / 131 (128 x 128, 16-bit 16x16x32 kernel, four- / two-stage ring), 192 (256 x 192, 16-bit), 193 (256 x 128, 16-bit) or 256");
    c->force_tile = tile;
    return AIDN_OK;
}

AIDN_API int aidn_mi355_set_attention_fast_path(void* ctx, int enabled)
{
    if (!ctx) return AIDN_ERR_INVALID_ARGUMENT;
    ((Ctx*)ctx)->attn_fast_path = (enabled == 2 || enabled == 3) ? enabled : (enabled != 0);
    return AIDN_OK;
}

// workspace of the fp32 paths that need one: small M (M <= 8, B [K,N]) and split-K partials; mode 0 B [K,N], 1 B [N,K], 2 fp16
// weights (small M only).  *ws stays null when no such path applies or a tile size is forced
static int smallm_ws(Ctx* c, void* stream, int M, int N, int K, int transB, void** ws, size_t* ws_bytes)
{
    *ws = nullptr; *ws_bytes = 0;
    if (c->force_tile != 0) return 0;
    size_t need = transB == 2 ? aidn::gemm_smallm_workspace_bytes(M, N, K) : aidn::gemm_f32_workspace_bytes(M, N, K, transB);
    if (!need) return 0;
    const int st = acquire_ws(c, stream, need, ws);
    // a stream under capture whose workspace would have to grow: the tiled kernel needs none
    if (st == AIDN_ERR_WORKSPACE) { *ws = nullptr; return 0; }
    if (st == 0) *ws_bytes = need;
    return st;
}

AIDN_API int aidn_mi355_sgemm(void* ctx, void* stream, const float* A, const float* B, float* C,
                     int M, int N, int K, float alpha, float beta, int transB)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!A || !B || !C) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "sgemm: A, B and C must not be null");
    if (M <= 0 || N <= 0 || K <= 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "sgemm: dimensions must be positive");
    int tile = c->force_tile;
    void* ws = nullptr; size_t ws_bytes = 0;
    if (int st = smallm_ws(c, stream, M, N, K, transB != 0, &ws, &ws_bytes)) return st;
    return hip_status(c, aidn::gemm_f32((hipStream_t)stream, A, B, C, M, N, K, alpha, beta, transB != 0, 1, 0, 0, 0, tile, nullptr, 0, 0.0f, ws,
                                        nullptr, ws_bytes), "gemm_f32");
}

AIDN_API int aidn_mi355_sgemm_batched(void* ctx, void* stream, const float* A, const float* B, float* C,
                             int M, int N, int K, int batch, float alpha, float beta)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!A || !B || !C) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "sgemm_batched: A, B and C must not be null");
    if (M <= 0 || N <= 0 || K <= 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "sgemm_batched: dimensions must be positive");
    if (batch <= 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "sgemm_batched: batch count must be positive");
    if (batch > 65535) return fail(c, AIDN_ERR_UNSUPPORTED, "sgemm_batched: more than 65535 batches");
    int tile = c->force_tile;
    return hip_status(c, aidn::gemm_f32((hipStream_t)stream, A, B, C, M, N, K, alpha, beta, 0, batch,
                                        (long long)M * K, (long long)K * N, (long long)M * N, tile), "gemm_f32 (batched)");
}

AIDN_API int aidn_mi355_sgemm_bias_act(void* ctx, void* stream, const float* A, const float* B, const float* bias, float* C,
                              int M, int N, int K, int activation, float act_param)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!A || !B || !C) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "sgemm_bias_act: A, B and C must not be null");
    if (M <= 0 || N <= 0 || K <= 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "sgemm_bias_act: dimensions must be positive");
    if (!valid_activation(activation)) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "sgemm_bias_act: unknown activation");
    int tile = c->force_tile;
    void* ws = nullptr; size_t ws_bytes = 0;
    if (int st = smallm_ws(c, stream, M, N, K, 0, &ws, &ws_bytes)) return st;
    return hip_status(c, aidn::gemm_f32((hipStream_t)stream, A, B, C, M, N, K, 1.0f, 0.0f, 0, 1, 0, 0, 0, tile, bias, activation, act_param, ws,
                                        nullptr, ws_bytes), "gemm_f32 (bias + activation)");
}
AIDN_API int aidn_mi355_sgemm_f16weight(void* ctx, void* stream, const float* A, const uint16_t* B_f16, const float* bias, float* C,
                               int M, int N, int K, int activation, float act_param)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!A || !B_f16 || !C) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "sgemm_f16weight: A, B and C must not be null");
    if (M <= 0 || N <= 0 || K <= 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "sgemm_f16weight: dimensions must be positive");
    if (!valid_activation(activation)) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "sgemm_f16weight: unknown activation");
    void* ws = nullptr; size_t ws_bytes = 0;
    if (int st = smallm_ws(c, stream, M, N, K, 2, &ws, &ws_bytes)) return st;
    return hip_status(c, aidn::gemm_f32_f16weight((hipStream_t)stream, A, B_f16, C, M, N, K, c->force_tile, bias, activation, act_param, ws,
                                                  ws_bytes), "gemm_f32_f16weight");
}
AIDN_API int aidn_mi355_hgemm_bias_act(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, const float* bias, void* C,
                              int out_is_f32, int M, int N, int K, int activation, float act_param)
{ return gemm16_common(ctx, stream, 0, A, B, C, out_is_f32 != 0, M, N, K, bias, activation, act_param); }
AIDN_API int aidn_mi355_bf16gemm_bias_act(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, const float* bias, void* C,
                                 int out_is_f32, int M, int N, int K, int activation, float act_param)
{ return gemm16_common(ctx, stream, 1, A, B, C, out_is_f32 != 0, M, N, K, bias, activation, act_param); }

// ---- pre-packed weight operand: kind 0 fp32 (B [K,N], or [N,K] with transB), 1 fp16, 2 bf16 (B [K,N])
AIDN_API uint64_t aidn_mi355_packed_b_bytes(int kind, int K, int N, int transB)
{
    if (kind == 0) return aidn::gemm_f32_packed_b_bytes(N, K, transB != 0);
    if ((kind == 1 || kind == 2) && !transB) return aidn::gemm_16_packed_b_bytes(N, K);
    return 0;
}
AIDN_API int aidn_mi355_pack_b(void* ctx, void* stream, int kind, const void* B, int K, int N, int transB, void* packed)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!B || !packed) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "pack_b: B and packed must not be null");
    if (K <= 0 || N <= 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "pack_b: dimensions must be positive");
    if (kind < 0 || kind > 2 || (kind != 0 && transB)) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "pack_b: kind 0 (fp32), 1 (fp16) or 2 (bf16); transB only for fp32");
    if (aidn_mi355_packed_b_bytes(kind, K, N, transB) == 0) return fail(c, AIDN_ERR_UNSUPPORTED, "pack_b: dimensions beyond the packed layout");
    if ((((uintptr_t)packed) & 15u) != 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "pack_b: packed must be 16-byte aligned");
    if (kind == 0) return hip_status(c, aidn::gemm_f32_pack_b((hipStream_t)stream, (const float*)B, K, N, transB != 0, packed), "pack_b");
    return hip_status(c, aidn::gemm_16_pack_b((hipStream_t)stream, (const uint16_t*)B, K, N, packed), "pack_b");
}
AIDN_API int aidn_mi355_gemm_packed_b(void* ctx, void* stream, int kind, const void* A, const void* packedB, const float* bias, void* C,
                             int out_is_f32, int M, int N, int K, int transB, int activation, float act_param)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!A || !packedB || !C) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm_packed_b: A, packedB and C must not be null");
    if (M <= 0 || N <= 0 || K <= 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm_packed_b: dimensions must be positive");
    if (kind < 0 || kind > 2 || (kind != 0 && transB)) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm_packed_b: kind 0 (fp32), 1 (fp16) or 2 (bf16); transB only for fp32");
    if (!valid_activation(activation)) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm_packed_b: unknown activation");
    if (aidn_mi355_packed_b_bytes(kind, K, N, transB) == 0) return fail(c, AIDN_ERR_UNSUPPORTED, "gemm_packed_b: dimensions beyond the packed layout");
    if (((((uintptr_t)packedB) | ((uintptr_t)C)) & 15u) != 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm_packed_b: packedB and C must be 16-byte aligned");
    void* ws = nullptr;
    const size_t need = kind == 0 ? aidn::gemm_f32_packed_workspace_bytes(M, N, K, transB != 0) : aidn::gemm_16_packed_workspace_bytes(M, N, K);
    if (kind != 0 && need == 0) return fail(c, AIDN_ERR_UNSUPPORTED, "gemm_packed_b: problem beyond the 4 GiB workspace limit");
    if (need) {
        if (int st = acquire_ws(c, stream, need, &ws)) return st;       // (a stream under capture must have it reserved: B itself is not at hand)
    }
    if (kind == 0) {
        if ((((uintptr_t)A) & 15u) != 0 && K % 32 == 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "gemm_packed_b: A must be 16-byte aligned");
        return hip_status(c, aidn::gemm_f32((hipStream_t)stream, (const float*)A, nullptr, (float*)C, M, N, K, 1.0f, 0.0f, transB != 0, 1, 0, 0, 0, 0,
                                            bias, activation, act_param, ws, (const float*)packedB, ws ? need : 0), "gemm_f32 (packed B)");
    }
    return hip_status(c, aidn::gemm_16((hipStream_t)stream, kind - 1, (const uint16_t*)A, nullptr, C, out_is_f32 != 0, M, N, K, 0, ws, ws ? need : 0,
                                       bias, activation, act_param, (const uint16_t*)packedB), "gemm_16 (packed B)");
}

AIDN_API int aidn_mi355_hgemm_f32out(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, float* C, int M, int N, int K)
{ return gemm16_common(ctx, stream, 0, A, B, C, 1, M, N, K); }
AIDN_API int aidn_mi355_hgemm_f16out(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K)
{ return gemm16_common(ctx, stream, 0, A, B, C, 0, M, N, K); }
AIDN_API int aidn_mi355_bf16gemm_f32out(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, float* C, int M, int N, int K)
{ return gemm16_common(ctx, stream, 1, A, B, C, 1, M, N, K); }
AIDN_API int aidn_mi355_bf16gemm_bf16out(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K)
{ return gemm16_common(ctx, stream, 1, A, B, C, 0, M, N, K); }

AIDN_API int aidn_mi355_hgemm_rope(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K,
                                   const float* cos_cache, const float* sin_cache, int head_dim, int rope_cols, int seq_len, int start_position)
{ return gemm16_rope_common(ctx, stream, 0, A, B, C, M, N, K, cos_cache, sin_cache, head_dim, rope_cols, seq_len, start_position); }
AIDN_API int aidn_mi355_bf16gemm_rope(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K,
                                      const float* cos_cache, const float* sin_cache, int head_dim, int rope_cols, int seq_len, int start_position)
{ return gemm16_rope_common(ctx, stream, 1, A, B, C, M, N, K, cos_cache, sin_cache, head_dim, rope_cols, seq_len, start_position); }

AIDN_API int aidn_mi355_convert_f32_to_f16(void* ctx, void* stream, const float* in, uint16_t* out, int64_t n)
{ return convert_common(ctx, stream, 0, in, out, n); }
AIDN_API int aidn_mi355_convert_f16_to_f32(void* ctx, void* stream, const uint16_t* in, float* out, int64_t n)
{ return convert_common(ctx, stream, 1, in, out, n); }
AIDN_API int aidn_mi355_convert_f32_to_bf16(void* ctx, void* stream, const float* in, uint16_t* out, int64_t n)
{ return convert_common(ctx, stream, 2, in, out, n); }
AIDN_API int aidn_mi355_convert_bf16_to_f32(void* ctx, void* stream, const uint16_t* in, float* out, int64_t n)
{ return convert_common(ctx, stream, 3, in, out, n); }

AIDN_API int aidn_mi355_attn_fwd_f32(void* ctx, void* stream, const aidn_attn_desc* desc, const float* q, const float* k, const float* v,
                            float* o, float* lse, const float* bias, const float* mask, float* weights)
{ return attn_common(ctx, stream, 0, desc, q, k, v, o, lse, bias, mask, weights); }
AIDN_API int aidn_mi355_attn_fwd_f16(void* ctx, void* stream, const aidn_attn_desc* desc, const uint16_t* q, const uint16_t* k, const uint16_t* v,
                            void* o, float* lse, const float* bias, const float* mask, float* weights)
{ return attn_common(ctx, stream, 1, desc, q, k, v, o, lse, bias, mask, weights); }
AIDN_API int aidn_mi355_attn_fwd_bf16(void* ctx, void* stream, const aidn_attn_desc* desc, const uint16_t* q, const uint16_t* k, const uint16_t* v,
                             void* o, float* lse, const float* bias, const float* mask, float* weights)
{ return attn_common(ctx, stream, 2, desc, q, k, v, o, lse, bias, mask, weights); }

AIDN_API int aidn_mi355_paged_attn_decode_f32(void* ctx, void* stream, const float* q, const float* kcache, const float* vcache,
                                     const int32_t* block_table, float* o, int heads, int kv_heads, int head_dim, int block_size,
                                     int seq_len, float scale, int splits)
{ return paged_common(ctx, stream, 0, q, kcache, vcache, block_table, o, heads, kv_heads, head_dim, block_size, 1, seq_len, 0, scale, splits, true); }
AIDN_API int aidn_mi355_paged_attn_decode_f16(void* ctx, void* stream, const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache,
                                     const int32_t* block_table, float* o, int heads, int kv_heads, int head_dim, int block_size,
                                     int seq_len, float scale, int splits)
{ return paged_common(ctx, stream, 1, q, kcache, vcache, block_table, o, heads, kv_heads, head_dim, block_size, 1, seq_len, 0, scale, splits, true); }
AIDN_API int aidn_mi355_paged_attn_decode_bf16(void* ctx, void* stream, const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache,
                                      const int32_t* block_table, float* o, int heads, int kv_heads, int head_dim, int block_size,
                                      int seq_len, float scale, int splits)
{ return paged_common(ctx, stream, 2, q, kcache, vcache, block_table, o, heads, kv_heads, head_dim, block_size, 1, seq_len, 0, scale, splits, true); }
AIDN_API int aidn_mi355_paged_attn_prefill_f32(void* ctx, void* stream, const float* q, const float* kcache, const float* vcache,
                                      const int32_t* block_table, float* o, int heads, int kv_heads, int head_dim, int block_size,
                                      int num_queries, int start_pos, float scale)
{
    long long key_len = (long long)start_pos + num_queries;
    if (key_len > 0x7FFFFFFFLL) return AIDN_ERR_INVALID_ARGUMENT;
    return paged_common(ctx, stream, 0, q, kcache, vcache, block_table, o, heads, kv_heads, head_dim, block_size, num_queries, (int)key_len,
                        start_pos, scale, 0, false);
}
AIDN_API int aidn_mi355_paged_attn_prefill_f16(void* ctx, void* stream, const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache,
                                      const int32_t* block_table, float* o, int heads, int kv_heads, int head_dim, int block_size,
                                      int num_queries, int start_pos, float scale)
{
    long long key_len = (long long)start_pos + num_queries;
    if (key_len > 0x7FFFFFFFLL) return AIDN_ERR_INVALID_ARGUMENT;
    return paged_common(ctx, stream, 1, q, kcache, vcache, block_table, o, heads, kv_heads, head_dim, block_size, num_queries, (int)key_len,
                        start_pos, scale, 0, false);
}
AIDN_API int aidn_mi355_paged_attn_prefill_bf16(void* ctx, void* stream, const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache,
                                       const int32_t* block_table, float* o, int heads, int kv_heads, int head_dim, int block_size,
                                       int num_queries, int start_pos, float scale)
{
    long long key_len = (long long)start_pos + num_queries;
    if (key_len > 0x7FFFFFFFLL) return AIDN_ERR_INVALID_ARGUMENT;
    return paged_common(ctx, stream, 2, q, kcache, vcache, block_table, o, heads, kv_heads, head_dim, block_size, num_queries, (int)key_len,
                        start_pos, scale, 0, false);
}

AIDN_API int aidn_mi355_rope_interleaved_f32(void* ctx, void* stream, const float* input, const float* cos_cache, const float* sin_cache,
                                    float* output, int64_t rows, int head_dim, int seq_len, int start_position)
{ return rope_common(ctx, stream, 0, input, cos_cache, sin_cache, output, rows, head_dim, seq_len, start_position); }
AIDN_API int aidn_mi355_rope_interleaved_f16(void* ctx, void* stream, const uint16_t* input, const float* cos_cache, const float* sin_cache,
                                    uint16_t* output, int64_t rows, int head_dim, int seq_len, int start_position)
{ return rope_common(ctx, stream, 1, input, cos_cache, sin_cache, output, rows, head_dim, seq_len, start_position); }
AIDN_API int aidn_mi355_rope_interleaved_bf16(void* ctx, void* stream, const uint16_t* input, const float* cos_cache, const float* sin_cache,
                                     uint16_t* output, int64_t rows, int head_dim, int seq_len, int start_position)
{ return rope_common(ctx, stream, 2, input, cos_cache, sin_cache, output, rows, head_dim, seq_len, start_position); }

AIDN_API int aidn_mi355_mha_fwd_f32(void* ctx, void* stream, const float* input, const float* wq, const float* wk, const float* wv,
                           const float* wo, const float* mask, int mask_mode, float* output, int B, int S, int dModel, int heads)
{ return mha_common(ctx, stream, 0, input, wq, wk, wv, nullptr, wo, mask, mask_mode, output, B, S, dModel, heads); }
AIDN_API int aidn_mi355_mha_fwd_f16(void* ctx, void* stream, const uint16_t* input, const uint16_t* wq, const uint16_t* wk, const uint16_t* wv,
                           const uint16_t* wo, const float* mask, int mask_mode, uint16_t* output, int B, int S, int dModel, int heads)
{ return mha_common(ctx, stream, 1, input, wq, wk, wv, nullptr, wo, mask, mask_mode, output, B, S, dModel, heads); }
AIDN_API int aidn_mi355_mha_fwd_bf16(void* ctx, void* stream, const uint16_t* input, const uint16_t* wq, const uint16_t* wk, const uint16_t* wv,
                            const uint16_t* wo, const float* mask, int mask_mode, uint16_t* output, int B, int S, int dModel, int heads)
{ return mha_common(ctx, stream, 2, input, wq, wk, wv, nullptr, wo, mask, mask_mode, output, B, S, dModel, heads); }

AIDN_API int aidn_mi355_mha_pack_qkv(void* ctx, void* stream, const void* wq, const void* wk, const void* wv, void* packed,
                                     int dModel, int elem_bytes)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    if (!wq || !wk || !wv || !packed) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "mha_pack_qkv: buffers must not be null");
    if (dModel <= 0) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "mha_pack_qkv: dModel must be positive");
    if (elem_bytes != 2 && elem_bytes != 4) return fail(c, AIDN_ERR_INVALID_ARGUMENT, "mha_pack_qkv: elem_bytes must be 2 or 4");
    return hip_status(c, gather_qkv((hipStream_t)stream, wq, wk, wv, packed, dModel, (size_t)elem_bytes), "mha_pack_qkv");
}
AIDN_API int aidn_mi355_mha_fwd_packed_f32(void* ctx, void* stream, const float* input, const float* wqkv, const float* wo,
                                           const float* mask, int mask_mode, float* output, int B, int S, int dModel, int heads)
{
    if (ctx && !wqkv) return fail((Ctx*)ctx, AIDN_ERR_INVALID_ARGUMENT, "mha (packed): the packed weight must not be null");
    return mha_common(ctx, stream, 0, input, nullptr, nullptr, nullptr, wqkv, wo, mask, mask_mode, output, B, S, dModel, heads);
}
AIDN_API int aidn_mi355_mha_fwd_packed_f16(void* ctx, void* stream, const uint16_t* input, const uint16_t* wqkv, const uint16_t* wo,
                                           const float* mask, int mask_mode, uint16_t* output, int B, int S, int dModel, int heads)
{
    if (ctx && !wqkv) return fail((Ctx*)ctx, AIDN_ERR_INVALID_ARGUMENT, "mha (packed): the packed weight must not be null");
    return mha_common(ctx, stream, 1, input, nullptr, nullptr, nullptr, wqkv, wo, mask, mask_mode, output, B, S, dModel, heads);
}
AIDN_API int aidn_mi355_mha_fwd_packed_bf16(void* ctx, void* stream, const uint16_t* input, const uint16_t* wqkv, const uint16_t* wo,
                                            const float* mask, int mask_mode, uint16_t* output, int B, int S, int dModel, int heads)
{
    if (ctx && !wqkv) return fail((Ctx*)ctx, AIDN_ERR_INVALID_ARGUMENT, "mha (packed): the packed weight must not be null");
    return mha_common(ctx, stream, 2, input, nullptr, nullptr, nullptr, wqkv, wo, mask, mask_mode, output, B, S, dModel, heads);
}

AIDN_API int aidn_mi355_reserve_workspace(void* ctx, void* stream, uint64_t bytes)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    void* ws = nullptr;
    return acquire_ws(c, stream, (size_t)bytes, &ws);
}
AIDN_API int aidn_mi355_release_stream_workspace(void* ctx, void* stream)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    WsSlot slot;
    {
        std::lock_guard<std::mutex> g(c->mu);
        auto it = c->ws.find(stream);
        if (it == c->ws.end()) return AIDN_OK;
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing((hipStream_t)stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone) {
            c->last_error = "release_stream_workspace: the stream is being captured";
            return AIDN_ERR_WORKSPACE;
        }
        slot = it->second;
        c->ws.erase(it);
    }
    // everything the library queued on this stream has to be through with the blocks before they go back
    if (hipError_t e = hipStreamSynchronize((hipStream_t)stream)) return hip_status(c, e, "release_stream_workspace");
    for (void* p : slot.retired) (void)hipFree(p);
    if (slot.cur) (void)hipFree(slot.cur);
    return AIDN_OK;
}
AIDN_API uint64_t aidn_mi355_workspace_bytes(void* ctx, void* stream)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return 0;
    std::lock_guard<std::mutex> g(c->mu);
    auto it = c->ws.find(stream);
    return it == c->ws.end() ? 0 : (uint64_t)it->second.bytes;
}

AIDN_API int aidn_mi355_attn_decode_f32(void* ctx, void* stream, const aidn_attn_desc* desc, const float* q, const float* k, const float* v,
                               float* o, float* lse, int splits)
{ return decode_common(ctx, stream, 0, desc, q, k, v, o, lse, splits); }
AIDN_API int aidn_mi355_attn_decode_f16(void* ctx, void* stream, const aidn_attn_desc* desc, const uint16_t* q, const uint16_t* k, const uint16_t* v,
                               void* o, float* lse, int splits)
{ return decode_common(ctx, stream, 1, desc, q, k, v, o, lse, splits); }
AIDN_API int aidn_mi355_attn_decode_bf16(void* ctx, void* stream, const aidn_attn_desc* desc, const uint16_t* q, const uint16_t* k, const uint16_t* v,
                                void* o, float* lse, int splits)
{ return decode_common(ctx, stream, 2, desc, q, k, v, o, lse, splits); }


// Allocation-free form of aidn_mi355_attn_decode_bf16: the split-KV partials live in the static device array `scratch`
// (through its per-device address), so the call never touches hipMalloc / hipFree.
AIDN_API int aidn_mi355_attn_decode_bf16_noalloc(void* ctx, void* stream, const aidn_attn_desc* desc, const uint16_t* q, const uint16_t* k,
                                                 const uint16_t* v, void* o, float* lse, int splits)
{
    Ctx* c = (Ctx*)ctx;
    if (!c) return AIDN_ERR_INVALID_ARGUMENT;
    void* ptr = c->device < kMaxDevices ? g_scratch_ptr[c->device] : nullptr;
    if (!ptr) return fail(c, AIDN_ERR_UNSUPPORTED, "decode (allocation-free): no static scratch buffer on this device");
    return decode_common(ctx, stream, 2, desc, q, k, v, o, lse, splits, ptr, kStaticScratchBytes);
}

}  // extern "C"
