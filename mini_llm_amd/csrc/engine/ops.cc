#include "ops.h"

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>

#include "kernels.h"

namespace minillm {

const char* dtype_name(int dt) { return dt == F32 ? "float32" : dt == BF16 ? "bfloat16" : "unknown dtype"; }

void fail(const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    throw OpError(buf);
}

static void check(int rc, const char* what) {
    if (rc == 0) return;
    if (rc < 0) fail("%s: the kernel refuses these sizes (code %d)", what, rc);
    fail("%s: HIP error %d (%s) at launch", what, rc, hipGetErrorString(static_cast<hipError_t>(rc)));
}

static void need_dtype(const Tensor2& t, const char* name) {
    if (t.dtype != F32 && t.dtype != BF16) fail("%s: unsupported dtype code %d (float32 or bfloat16)", name, t.dtype);
    if (t.data == nullptr && t.rows * t.cols > 0) fail("%s: null data pointer", name);
}

static bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// ---------------------------------------------------------------------------------------------
// scratch
// ---------------------------------------------------------------------------------------------
namespace {
struct Buffer {
    void* ptr = nullptr;
    size_t bytes = 0;
};
struct Key {
    int device;
    hipStream_t stream;
    std::string name;
    bool operator<(const Key& o) const {
        if (device != o.device) return device < o.device;
        if (stream != o.stream) return std::less<const void*>()(stream, o.stream);
        return name < o.name;
    }
};
std::mutex g_scratch_mutex;
std::map<Key, Buffer> g_scratch;
constexpr size_t GEMM_WORKSPACE_BYTES = 16 * 1024 + 256 * 1024;   // counters, then 1 KB per workgroup of a shared-tile launch
constexpr int DECODE_MAX_SPLIT = 8;

int current_device() {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) fail("hipGetDevice: %s", hipGetErrorString(e));
    return dev;
}

// Grows only; a fresh buffer is cleared when `zero` (kernels that use counters leave them at zero).
void* scratch(const char* name, size_t bytes, bool zero, hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    Buffer& b = g_scratch[Key{current_device(), stream, name}];
    if (b.ptr != nullptr && b.bytes >= bytes) return b.ptr;
    void* fresh = nullptr;
    hipError_t e = hipMalloc(&fresh, bytes);
    if (e != hipSuccess) fail("scratch '%s': hipMalloc of %zu bytes failed: %s", name, bytes, hipGetErrorString(e));
    if (zero) {
        // (the fill runs on the null stream, which a non-blocking stream does not wait for: the device is
        // synchronised so that no kernel on `stream` meets counters that are still being cleared)
        e = hipMemset(fresh, 0, bytes);
        if (e == hipSuccess) e = hipDeviceSynchronize();
        if (e != hipSuccess) fail("scratch '%s': clearing it failed: %s", name, hipGetErrorString(e));
    }
    if (b.ptr != nullptr) {
        // work queued with the old buffer may still run: wait for it, then free
        (void)hipDeviceSynchronize();
        (void)hipFree(b.ptr);
    }
    b.ptr = fresh;
    b.bytes = bytes;
    return fresh;
}

float* argmax_values(size_t n, hipStream_t s) { return static_cast<float*>(scratch("argmax_values", std::max<size_t>(n, 4096) * 4, false, s)); }
int* argmax_indices(size_t n, hipStream_t s) { return static_cast<int*>(scratch("argmax_indices", std::max<size_t>(n, 4096) * 4, false, s)); }
float* decode_partials(size_t n, hipStream_t s) { return static_cast<float*>(scratch("decode_partials", std::max<size_t>(n, 1 << 16) * 4, false, s)); }
int* decode_counters(size_t n, hipStream_t s) { return static_cast<int*>(scratch("decode_counters", std::max<size_t>(n, 4096) * 4, true, s)); }
void* gemm_workspace(hipStream_t s) { return scratch("gemm_workspace", GEMM_WORKSPACE_BYTES, true, s); }
}  // namespace

void reserve_attention_scratch(int rows, int n_heads, int head_dim, hipStream_t stream) {
    if (rows < 1 || n_heads < 1 || head_dim < 1) return;
    // (every launch shape keeps pairs x splits within max(8 x pairs, 256))
    decode_partials(std::max<size_t>(static_cast<size_t>(rows) * n_heads * DECODE_MAX_SPLIT, 256) * (head_dim + 2), stream);
    decode_counters(static_cast<size_t>(rows) * n_heads, stream);
}

void reserve_sampling_scratch(int rows, int vocab, hipStream_t stream) {
    const size_t chunks = static_cast<size_t>(mllm_argmax_chunks(vocab));
    argmax_values(std::max(rows, 1) * chunks, stream);
    argmax_indices(std::max(rows, 1) * chunks, stream);
}

void reserve_linear_scratch(hipStream_t stream) { gemm_workspace(stream); }

void release_scratch(hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    const int dev = current_device();
    bool any = false;
    for (auto it = g_scratch.begin(); it != g_scratch.end();) {
        if (it->first.device == dev && it->first.stream == stream) {
            if (!any) { (void)hipStreamSynchronize(stream); any = true; }
            (void)hipFree(it->second.ptr);
            it = g_scratch.erase(it);
        } else {
            ++it;
        }
    }
}

void* scratch_address(const char* name, hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    auto it = g_scratch.find(Key{current_device(), stream, name});
    return it == g_scratch.end() ? nullptr : it->second.ptr;
}

size_t scratch_bytes() {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    const int dev = current_device();
    size_t n = 0;
    for (const auto& kv : g_scratch)
        if (kv.first.device == dev) n += kv.second.bytes;
    return n;
}

Tuning& tuning() {
    static Tuning t;
    return t;
}

// ---------------------------------------------------------------------------------------------
// elementwise
// ---------------------------------------------------------------------------------------------
void embed(const int* ids, const int* positions, const Tensor2& wte, const Tensor2* wpe, const Tensor2& out,
           hipStream_t stream, const FedTokens* fed) {
    need_dtype(wte, "wte");
    const int T = static_cast<int>(out.rows), D = static_cast<int>(wte.cols);
    if (!wte.contiguous()) fail("embed: wte must be contiguous");
    if (out.dtype != F32 || out.cols != D || !out.contiguous()) fail("embed: out must be contiguous float32 [%d, %d]", T, D);
    const void* table = nullptr;
    if (wpe != nullptr && wpe->data != nullptr) {
        if (positions == nullptr) fail("embed: positions are needed with a position table");
        if (wpe->dtype != wte.dtype || wpe->cols != D || !wpe->contiguous())
            fail("embed: wpe must be contiguous [P, %d] in wte's dtype", D);
        table = wpe->data;
    }
    const bool feeds = fed != nullptr && fed->src != nullptr;
    if (feeds && (fed->prev == nullptr || fed->n_prev < 1)) fail("embed: fed tokens need the earlier step's sampled tokens");
    check(mllm_embed(ids, table ? positions : nullptr, wte.data, table, static_cast<float*>(out.data), T, D, wte.dtype,
                     feeds ? fed->src : nullptr, feeds ? fed->prev : nullptr, feeds ? fed->n_prev : 0, stream), "embed");
}

void select_tokens(int* ids, const int* src, const int* prev, int n, int n_prev, hipStream_t stream) {
    check(mllm_select_tokens(ids, src, prev, n, n_prev, stream), "select_tokens");
}

void reset_state(void* state, size_t slot_bytes, int n_slots, const int* slots, const int* starts, int n_seqs,
                 hipStream_t stream) {
    const int rc = mllm_reset_state(state, slot_bytes, n_slots, slots, starts, n_seqs, stream);
    if (rc == -1) fail("reset_state: a slot of %zu bytes is no multiple of 4 bytes", slot_bytes);
    check(rc, "reset_state");
}

void layernorm(const Tensor2& x, const float* gamma, const float* beta, float eps, const Tensor2& out,
               const int* rows, hipStream_t stream) {
    need_dtype(out, "layernorm out");
    if (x.dtype != F32 || !x.contiguous()) fail("layernorm: input must be contiguous float32 [rows, D]");
    const int D = static_cast<int>(x.cols), n = static_cast<int>(out.rows);
    if (rows == nullptr && out.rows != x.rows) fail("layernorm: out has %lld rows, the input %lld", (long long)out.rows, (long long)x.rows);
    if (out.cols != D || !out.contiguous()) fail("layernorm: out must be contiguous [%d, %d]", n, D);
    if (gamma == nullptr) fail("layernorm: gamma is missing");
    check(mllm_layernorm(static_cast<const float*>(x.data), rows, gamma, beta, out.data, n, D, eps, out.dtype, stream),
          "layernorm");
}

static void check_pages(const Tensor2& k_pages, const Tensor2& v_pages, int dtype, const char* what) {
    if (k_pages.dtype != dtype || v_pages.dtype != dtype || !k_pages.contiguous() || !v_pages.contiguous() ||
        k_pages.cols != v_pages.cols || k_pages.rows != v_pages.rows)
        fail("%s: key and value pages must be contiguous [rows, kv_dim] %s of one shape", what, dtype_name(dtype));
}

void kv_append(const Tensor2& src, int k_col, int v_col, const Tensor2& k_pages, const Tensor2& v_pages,
               const int* slots, hipStream_t stream) {
    need_dtype(src, "kv_append src");
    check_pages(k_pages, v_pages, src.dtype, "kv_append");
    const int kv_dim = static_cast<int>(k_pages.cols);
    if (std::max(k_col, v_col) + kv_dim > src.cols || std::min(k_col, v_col) < 0)
        fail("kv_append: key/value columns lie outside the source rows");
    if (slots == nullptr) fail("kv_append: slots are missing");
    check(mllm_kv_append(src.data, static_cast<int>(src.stride), k_col, v_col, k_pages.data, v_pages.data, kv_dim, slots,
                         static_cast<int>(src.rows), src.dtype, stream), "kv_append");
}

// ---------------------------------------------------------------------------------------------
// products
// ---------------------------------------------------------------------------------------------
static int out_dtype_of(int epilogue, int act_dtype) {
    return (epilogue == ADD_RESIDUAL || epilogue == STORE_F32) ? F32 : act_dtype;
}

static void check_linear(int64_t M, int64_t K, int a_dtype, const Tensor2& w, const Tensor2& out, int epilogue,
                         const char* what) {
    need_dtype(w, "w");
    if (epilogue < STORE || epilogue > STORE_F32) fail("%s: unknown epilogue %d", what, epilogue);
    if (w.cols != K || w.dtype != a_dtype)
        fail("%s: a is [%lld, %lld] %s, w is [%lld, %lld] %s", what, (long long)M, (long long)K, dtype_name(a_dtype),
             (long long)w.rows, (long long)w.cols, dtype_name(w.dtype));
    const int want = out_dtype_of(epilogue, a_dtype);
    if (out.rows != M || out.cols != w.rows || out.dtype != want)
        fail("%s: out must be [%lld, %lld] %s, got [%lld, %lld] %s", what, (long long)M, (long long)w.rows, dtype_name(want),
             (long long)out.rows, (long long)out.cols, dtype_name(out.dtype));
}

// Whether the product kernel that runs for these rows writes keys and values to the pages in its epilogue.
static bool scatter_is_fused(int dtype, int64_t rows) { return dtype == BF16 && rows > 64; }

void linear(const Tensor2& a, const Tensor2& w, const float* bias, const Tensor2& out, int epilogue,
            const KvScatter* kv, hipStream_t stream) {
    need_dtype(a, "a");
    const int64_t M = a.rows, K = a.cols, N = w.rows;
    check_linear(M, K, a.dtype, w, out, epilogue, "linear");
    if (kv != nullptr) {
        if (epilogue != STORE) fail("linear: the key/value scatter needs the plain store");
        check_pages(kv->k_pages, kv->v_pages, a.dtype, "linear (key/value scatter)");
        const int kv_dim = static_cast<int>(kv->k_pages.cols);
        if (N != kv->q_cols + 2 * kv_dim) fail("linear: %lld columns are not %d + 2 x %d", (long long)N, kv->q_cols, kv_dim);
        if (!scatter_is_fused(a.dtype, M)) {
            linear(a, w, bias, out, epilogue, nullptr, stream);
            kv_append(out, kv->q_cols, kv->q_cols + kv_dim, kv->k_pages, kv->v_pages, kv->slots, stream);
            return;
        }
        if (kv->q_cols % 4 || kv_dim % 4) fail("linear: the query and key/value widths (%d, %d) must be multiples of 4", kv->q_cols, kv_dim);
    }
    int rc;
    if (a.dtype == F32) {
        rc = mllm_gemm_f32(static_cast<const float*>(a.data), static_cast<int>(a.stride), static_cast<const float*>(w.data),
                           static_cast<int>(w.stride), bias, out.data, static_cast<int>(out.stride), static_cast<int>(M),
                           static_cast<int>(N), static_cast<int>(K), epilogue, stream);
    } else if (kv != nullptr) {
        rc = mllm_gemm_bf16_kv(a.data, static_cast<int>(a.stride), w.data, static_cast<int>(w.stride), bias, out.data,
                               static_cast<int>(out.stride), static_cast<int>(M), static_cast<int>(N), static_cast<int>(K),
                               kv->slots, kv->k_pages.data, kv->v_pages.data, kv->q_cols, static_cast<int>(kv->k_pages.cols),
                               stream);
    } else {
        void* ws = M <= 256 ? gemm_workspace(stream) : nullptr;
        rc = mllm_gemm_bf16(a.data, static_cast<int>(a.stride), w.data, static_cast<int>(w.stride), bias, out.data,
                            static_cast<int>(out.stride), static_cast<int>(M), static_cast<int>(N), static_cast<int>(K),
                            epilogue, ws, ws ? GEMM_WORKSPACE_BYTES : 0, stream);
    }
    if (rc == -1 && a.dtype == BF16)
        fail("linear(bfloat16): K=%lld and the row strides (%lld, %lld) must be multiples of 8 elements and the operands "
             "16-byte aligned", (long long)K, (long long)a.stride, (long long)w.stride);
    check(rc, "linear");
}

void merge_splits(const AttentionSplits& a, const Tensor2& out, hipStream_t stream) {
    if (out.rows != a.n_tokens || out.cols != static_cast<int64_t>(a.n_heads) * a.head_dim)
        fail("merge_splits: out must be [%d, %d]", a.n_tokens, a.n_heads * a.head_dim);
    check(mllm_merge_attention_splits(a.ws, a.n_tokens, a.n_heads, a.head_dim, a.nsplit, out.data,
                                      static_cast<int>(out.stride), out.dtype, stream), "merge_splits");
}

void linear_from_splits(const AttentionSplits& a, const Tensor2& w, const float* bias, const Tensor2& out,
                        int epilogue, void* tmp, hipStream_t stream) {
    const int64_t M = a.n_tokens, K = static_cast<int64_t>(a.n_heads) * a.head_dim;
    check_linear(M, K, a.dtype, w, out, epilogue, "linear (merging attention splits)");
    if (a.dtype == BF16 && w.stride % 8 == 0 && aligned(w.data, 16)) {
        const int rc = mllm_gemm_bf16_merged(a.ws, a.ml(), a.nsplit, a.n_heads, a.head_dim, w.data, static_cast<int>(w.stride),
                                             bias, out.data, static_cast<int>(out.stride), static_cast<int>(M),
                                             static_cast<int>(w.rows), epilogue, stream);
        if (rc == 0) return;
        if (rc != -2) check(rc, "linear (merging attention splits)");
    }
    if (tmp == nullptr) fail("linear (merging attention splits): these sizes need a buffer for the merged rows");
    Tensor2 merged(tmp, a.dtype, M, K);
    merge_splits(a, merged, stream);
    linear(merged, w, bias, out, epilogue, nullptr, stream);
}

void ln_linear(const Tensor2& x, const float* gamma, const float* beta, float eps, const Tensor2& w,
               const float* bias, const Tensor2& out, int epilogue, const int* rows, void* tmp,
               const KvScatter* kv, hipStream_t stream) {
    const int64_t M = out.rows, K = x.cols;
    if (x.dtype != F32) fail("ln_linear: the input must be the float32 stream");
    check_linear(M, K, w.dtype, w, out, epilogue, "ln_linear");
    if (rows == nullptr && x.rows != M) fail("ln_linear: out has %lld rows, the input %lld", (long long)M, (long long)x.rows);
    // (More rows than that: the norm is a kernel of its own. Normalising in the tiled product while it stages
    // its rows was measured at 64 to 256 rows and lost: every workgroup of a row tile has to pull the tile's
    // fp32 rows through its own L1 for the statistics, 6.5 us at 64 rows of 768, more than the norm's kernel.)
    if (kv == nullptr && w.dtype == BF16 && M <= tuning().ln_fuse_max_rows && x.contiguous() && aligned(gamma, 16) &&
        (beta == nullptr || aligned(beta, 16))) {
        const int rc = mllm_ln_gemm_bf16(static_cast<const float*>(x.data), static_cast<int>(x.stride), rows, gamma, beta, eps,
                                         w.data, static_cast<int>(w.stride), bias, out.data, static_cast<int>(out.stride),
                                         static_cast<int>(M), static_cast<int>(w.rows), static_cast<int>(K), epilogue, stream);
        if (rc == 0) return;
        if (rc != -2) check(rc, "ln_linear");
    }
    if (tmp == nullptr) fail("ln_linear: these sizes need a buffer for the normalised rows");
    Tensor2 h(tmp, w.dtype, M, K);
    layernorm(x, gamma, beta, eps, h, rows, stream);
    linear(h, w, bias, out, epilogue, kv, stream);
}

// ---------------------------------------------------------------------------------------------
// attention
// ---------------------------------------------------------------------------------------------
// How many workgroups share one (token, head) pair's keys, and wavefronts per workgroup.
static void decode_launch_shape(int pairs, int max_ctx_len, bool unmerged, int* nsplit, int* waves, bool* merge_kernel) {
    const Tuning& t = tuning();
    *merge_kernel = false;
    if (t.decode_nsplit > 0) { *nsplit = t.decode_nsplit; *waves = t.decode_waves; return; }
    if (unmerged && !(t.long_context_splits && std::min(256 / std::max(pairs, 1), max_ctx_len / 512) >= 8)) {
        // The splits cost nothing to merge here (the next product does it while it loads), so few pairs
        // are spread over the compute units: a unit streams keys at 35 to 90 GB/s, and a pair's keys
        // and values at 768 tokens are 200 KB. Every split keeps at least 128 keys. (Measured at GPT-2
        // small sizes, 768 keys: 12 pairs x 4 splits of 4 wavefronts and 96 pairs x 2 splits of 8
        // wavefronts are the fastest shapes; more workgroups than compute units lose again.)
        if (t.unmerged_nsplit > 0) { *nsplit = t.unmerged_nsplit; *waves = t.unmerged_waves; return; }
        const int n = std::max(1, std::min({4, 256 / std::max(pairs, 1), max_ctx_len / 128}));
        if (n > 1) {
            const int keys = (max_ctx_len + n - 1) / n;
            *nsplit = n;
            *waves = std::max(2, std::min(12, (keys + 63) / 64));
            return;
        }
    }
    // Long contexts at few pairs (batch 1 to 3 at GPT-2 sizes): up to 4 workgroups a pair leave most of the
    // chip idle while each streams megabytes (12 pairs at 32,000 keys: 51 us a layer, 1.9 TB/s). They are
    // split over up to 256 workgroups, at least 512 keys each, and a small kernel merges the states: one
    // more launch, which pays from 8 splits on.
    if (t.long_context_splits) {
        const int n = std::min({256 / std::max(pairs, 1), max_ctx_len / 512, 64});
        if (n >= 8) {
            const int keys = (max_ctx_len + n - 1) / n;
            *nsplit = n;
            *waves = std::max(2, std::min(12, (keys + 63) / 64));
            *merge_kernel = true;
            return;
        }
    }
    // One workgroup per pair: merging splits in the kernel (fences, a second merge) costs about 3 us,
    // more than the parallelism gains below about 2,000 keys (measured at 12 to 96 pairs). Few pairs get
    // more wavefronts each instead (measured: 12 are 1 to 3 % of a decode step faster than 8 up to 200
    // pairs at GPT-2 small to XL sizes, 3 % slower from 384 pairs).
    *nsplit = 1;
    *waves = pairs >= 512 ? 4 : pairs > 256 ? 6 : 12;
}

static bool pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

bool paged_attention(const AttentionArgs& a, AttentionSplits* splits, hipStream_t stream) {
    need_dtype(a.q, "q");
    const int T = static_cast<int>(a.q.rows);
    const int kv_dim = a.n_kv_heads * a.head_dim, q_dim = a.n_heads * a.head_dim;
    const int esz = static_cast<int>(a.q.esz());
    if (a.n_heads < 1 || a.n_kv_heads < 1 || a.n_heads % a.n_kv_heads != 0)
        fail("paged_attention: n_heads=%d is not a multiple of n_kv_heads=%d", a.n_heads, a.n_kv_heads);
    if (a.head_dim % 8 != 0 || a.head_dim > 256) fail("paged_attention: head_dim=%d is not supported (multiples of 8 up to 256)", a.head_dim);
    if (a.q_col < 0 || a.q_col + q_dim > a.q.cols) fail("paged_attention: query columns lie outside q's rows");
    if (a.out.rows != T || a.out.cols != q_dim || a.out.dtype != a.q.dtype)
        fail("paged_attention: out must be [%d, %d] %s", T, q_dim, dtype_name(a.q.dtype));
    check_pages(a.k_pages, a.v_pages, a.q.dtype, "paged_attention");
    if (a.k_pages.cols != kv_dim) fail("paged_attention: the pages are %lld wide, %d expected", (long long)a.k_pages.cols, kv_dim);
    if (a.page_size < 1 || a.k_pages.rows % a.page_size != 0) fail("paged_attention: the page pool is not a whole number of pages");
    if (a.block_tables == nullptr || a.token_seq == nullptr || a.positions == nullptr || a.n_seqs < 1 || a.max_blocks < 1)
        fail("paged_attention: block tables, token_seq and positions are needed");
    if ((a.q.stride * esz) % 16 || (a.q_col * esz) % 16 || (a.head_dim * esz) % 16 || !aligned(a.q.data, 16))
        fail("paged_attention: query rows and heads must be 16-byte aligned");
    const int lpk = a.head_dim * esz / 16;
    const bool single_ok = lpk >= 2 && pow2(lpk) && pow2(a.page_size) && a.max_blocks <= 4096;
    const bool decode = a.max_q_len == 1 && single_ok;
    const int* slots = nullptr;
    if (a.append) {
        if (a.slots == nullptr) fail("paged_attention: append needs the tokens' page rows");
        if (!decode) {
            kv_append(a.q, a.k_col, a.v_col, a.k_pages, a.v_pages, a.slots, stream);
        } else {
            if (std::max(a.k_col, a.v_col) + kv_dim > a.q.cols || std::min(a.k_col, a.v_col) < 0 || (a.k_col * esz) % 16 ||
                (a.v_col * esz) % 16)
                fail("paged_attention: key/value columns lie outside q's rows or are not 16-byte aligned");
            slots = a.slots;
        }
    }
    // Prompt portions go to a kernel that shares key tiles among 64 queries: the bfloat16 matrix-core kernel at
    // its head and page sizes, otherwise the kernel that works in true 32-bit at any head size (multiples of 16)
    // and page size. What neither takes, and single tokens at sizes the decode kernel refuses, go to the
    // one-wavefront-per-query kernel.
    const bool have_tiles = a.max_q_len > 1 && a.cu_q != nullptr && a.ctx_len != nullptr;
    const bool tiles_ok = have_tiles && a.q.dtype == BF16 && (a.head_dim == 32 || a.head_dim == 64 || a.head_dim == 128) &&
                          pow2(a.page_size) && a.page_size >= a.head_dim / 16 && a.max_blocks <= 2048;
    const bool tiled_ok = have_tiles && !tiles_ok && a.head_dim % 16 == 0 && (kv_dim * esz) % 16 == 0 && (a.out.stride * esz) % 8 == 0 &&
                          aligned(a.out.data, 16) && aligned(a.k_pages.data, 16) && aligned(a.v_pages.data, 16);
    if (tiles_ok && (!aligned(a.out.data, 16) || (a.out.stride * esz) % 8)) fail("paged_attention: output rows must be 8-byte aligned");
    auto portions = [&](int first_seq) {
        const int B = a.n_seqs - first_seq, tiles = (T - first_seq) / 64 + B;      // (the leading sequences bring one row each)
        if (tiles_ok) {
            tuning().seen.prefill_tile_launches += 1;
            check(mllm_prefill_attention_bf16(a.q.data, static_cast<int>(a.q.stride), a.q_col, a.k_pages.data, a.v_pages.data, kv_dim,
                                              a.block_tables + static_cast<size_t>(first_seq) * a.max_blocks, a.max_blocks,
                                              a.cu_q + first_seq, a.ctx_len + first_seq, B, tiles, a.n_heads, a.n_kv_heads,
                                              a.head_dim, a.page_size, a.scale, a.window, a.out.data,
                                              static_cast<int>(a.out.stride), stream), "prefill_attention");
        } else {
            tuning().seen.tiled_f32_launches += 1;
            check(mllm_paged_attention_tiled(a.q.data, static_cast<int>(a.q.stride), a.q_col, a.k_pages.data, a.v_pages.data, kv_dim,
                                             a.block_tables + static_cast<size_t>(first_seq) * a.max_blocks, a.max_blocks,
                                             a.cu_q + first_seq, a.ctx_len + first_seq, B, tiles, a.n_heads, a.n_kv_heads,
                                             a.head_dim, a.page_size, a.scale, a.window, a.out.data,
                                             static_cast<int>(a.out.stride), a.q.dtype, stream), "paged_attention (tiles)");
        }
    };
    if ((tiles_ok || tiled_ok) && a.n_single > 0 && a.n_single < a.n_seqs) {
        // A mixed step: the leading single tokens, then the portions, two launches over disjoint rows
        // (every row's keys and values are in the pages by now). Row numbers in cu_q are absolute, so q
        // and out are passed whole and the per-sequence arrays from the first portion on.
        if (single_ok) {
            AttentionArgs d = a;
            d.q = a.q.row_range(0, a.n_single);
            d.out = a.out.row_range(0, a.n_single);
            d.n_seqs = a.n_single;
            d.max_q_len = 1;
            d.append = 0;
            d.may_split = 0;
            paged_attention(d, nullptr, stream);
        } else {
            tuning().seen.generic_attention_launches += 1;
            check(mllm_paged_attention_generic(a.q.data, static_cast<int>(a.q.stride), a.q_col, a.k_pages.data, a.v_pages.data, kv_dim,
                                               a.block_tables, a.max_blocks, a.token_seq, a.positions, a.n_single, a.n_heads,
                                               a.n_kv_heads, a.head_dim, a.page_size, a.scale, a.window, a.out.data,
                                               static_cast<int>(a.out.stride), a.q.dtype, stream), "paged_attention");
        }
        portions(a.n_single);
        return false;
    }
    if (decode) {
        const int pairs = T * a.n_heads;
        bool unmerged = a.may_split && splits != nullptr && a.q.dtype == BF16 && T <= tuning().merge_max_rows &&
                        a.head_dim % 8 == 0 && tuning().decode_nsplit == 0;
        int nsplit = 1, waves = 12;
        bool merge_kernel = false;
        decode_launch_shape(pairs, a.max_ctx_len, unmerged, &nsplit, &waves, &merge_kernel);
        unmerged = unmerged && nsplit > 1 && !merge_kernel;
        float* ws = decode_partials(nsplit > 1 ? static_cast<size_t>(pairs) * nsplit * (a.head_dim + 2) : 1, stream);
        int* counters = decode_counters(pairs, stream);
        // every sequence of the batch brings one token: token t is sequence t, and the kernel need not load that
        const int* seq_of_token = (a.n_single == T && T == a.n_seqs) ? nullptr : a.token_seq;
        check(mllm_decode_attention(a.q.data, static_cast<int>(a.q.stride), a.q_col, a.k_pages.data, a.v_pages.data, kv_dim,
                                    a.block_tables, a.max_blocks, seq_of_token, a.positions, T, a.n_heads, a.n_kv_heads,
                                    a.head_dim, a.page_size, a.scale, a.window, nsplit, waves, a.out.data,
                                    static_cast<int>(a.out.stride), ws, counters, a.k_col, a.v_col, slots,
                                    unmerged || merge_kernel ? 1 : 0, a.q.dtype, stream), "decode_attention");
        tuning().seen.max_decode_splits = std::max(tuning().seen.max_decode_splits, nsplit);
        if (merge_kernel) tuning().seen.merge_kernel_launches += 1;
        if (merge_kernel)
            check(mllm_merge_attention_splits(ws, T, a.n_heads, a.head_dim, nsplit, a.out.data, static_cast<int>(a.out.stride),
                                              a.q.dtype, stream), "merge_splits");
        if (unmerged) {
            splits->ws = ws;
            splits->n_tokens = T;
            splits->n_heads = a.n_heads;
            splits->head_dim = a.head_dim;
            splits->nsplit = nsplit;
            splits->dtype = a.q.dtype;
            return true;
        }
        return false;
    }
    if (tiles_ok || tiled_ok) {
        portions(0);
        return false;
    }
    tuning().seen.generic_attention_launches += 1;
    check(mllm_paged_attention_generic(a.q.data, static_cast<int>(a.q.stride), a.q_col, a.k_pages.data, a.v_pages.data, kv_dim,
                                       a.block_tables, a.max_blocks, a.token_seq, a.positions, T, a.n_heads, a.n_kv_heads,
                                       a.head_dim, a.page_size, a.scale, a.window, a.out.data, static_cast<int>(a.out.stride),
                                       a.q.dtype, stream), "paged_attention");
    return false;
}

// ---------------------------------------------------------------------------------------------
// sampling
// ---------------------------------------------------------------------------------------------
void argmax(const Tensor2& logits, int* out, hipStream_t stream, int* mirror) {
    if (logits.dtype != F32) fail("argmax: logits must be float32");
    const int n = static_cast<int>(logits.rows), V = static_cast<int>(logits.cols);
    const size_t chunks = static_cast<size_t>(mllm_argmax_chunks(V));
    float* pv = argmax_values(n * chunks, stream);
    int* pi = argmax_indices(n * chunks, stream);
    check(mllm_argmax_mirrored(static_cast<const float*>(logits.data), static_cast<int>(logits.stride), n, V, out, mirror, pv, pi, stream), "argmax");
}

void sample(const Tensor2& logits, const float* temperature, const float* u, int* out, hipStream_t stream, int* mirror) {
    if (logits.dtype != F32) fail("sample: logits must be float32");
    if (temperature == nullptr || u == nullptr) fail("sample: temperatures and uniform numbers are needed");
    check(mllm_sample_mirrored(static_cast<const float*>(logits.data), static_cast<int>(logits.stride), static_cast<int>(logits.rows),
                      static_cast<int>(logits.cols), temperature, u, out, mirror, stream), "sample");
}

}  // namespace minillm
