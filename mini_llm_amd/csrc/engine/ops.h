// The engine's device operations: checked dispatch over the HIP kernels.
//
// Every op checks on the host that shapes, strides and dtypes are what the kernel it picks and
// that kernel's grid assume, chooses among the kernels of an operation by size, and launches on
// the stream it is given. A refusal is an OpError
// with a message that names the sizes. There is no CPU path.
//
// The parts (parts.h) and, through the C ABI, the kernel tests (kernels/ops.py) call the same
// functions, so the choice of kernels is made in one place.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <stdexcept>
#include <string>

namespace minillm {

enum DType : int { F32 = 0, BF16 = 1 };
inline size_t dtype_size(int dt) { return dt == F32 ? 4 : 2; }
const char* dtype_name(int dt);

enum Epilogue : int { STORE = 0, GELU_TANH = 1, GELU_ERF = 2, ADD_RESIDUAL = 3, STORE_F32 = 4 };

class OpError : public std::runtime_error {
public:
    explicit OpError(const std::string& what) : std::runtime_error(what) {}
};
[[noreturn]] void fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

// A 2-D view of device memory; the last dimension is contiguous, `stride` elements lie between rows.
struct Tensor2 {
    void* data = nullptr;
    int dtype = F32;
    int64_t rows = 0, cols = 0, stride = 0;

    Tensor2() = default;
    Tensor2(void* d, int dt, int64_t r, int64_t c) : data(d), dtype(dt), rows(r), cols(c), stride(c) {}
    Tensor2(void* d, int dt, int64_t r, int64_t c, int64_t s) : data(d), dtype(dt), rows(r), cols(c), stride(s) {}
    size_t esz() const { return dtype_size(dtype); }
    bool contiguous() const { return stride == cols; }
    Tensor2 row_range(int64_t first, int64_t n) const {
        return Tensor2(static_cast<char*>(data) + first * stride * static_cast<int64_t>(esz()), dtype, n, cols, stride);
    }
};

// Second destination of a fused QKV product: the columns after the first q_cols are keys, then
// values (kv_dim = k_pages.cols each); row m's also go to row slots[m] (>= 0) of the pages.
struct KvScatter {
    const int* slots = nullptr;
    Tensor2 k_pages, v_pages;
    int q_cols = 0;
};

// The output of decode attention that has not been merged yet: every (token, head) pair's keys were
// split over `nsplit` workgroups whose states lie in the attention scratch (layout:
// kernels/attention_decode.hip). `linear_from_splits` merges while it loads. Valid until the next
// attention launch on the same stream.
struct AttentionSplits {
    float* ws = nullptr;
    int n_tokens = 0, n_heads = 0, head_dim = 0, nsplit = 0, dtype = BF16;
    bool valid() const { return ws != nullptr; }
    float* ml() const { return ws + static_cast<size_t>(n_tokens) * n_heads * nsplit * head_dim; }
};

struct AttentionArgs {
    Tensor2 q;                     // [T, >= q_col + n_heads * head_dim]
    int q_col = 0, n_heads = 0, n_kv_heads = 0, head_dim = 0;
    Tensor2 k_pages, v_pages;      // [n_pages * page_size, n_kv_heads * head_dim]
    int page_size = 0;
    const int* block_tables = nullptr;     // [n_seqs, max_blocks]
    int n_seqs = 0, max_blocks = 0;
    const int* token_seq = nullptr;        // [T] row of block_tables
    const int* positions = nullptr;        // [T]
    float scale = 1.f;
    int window = 0;
    Tensor2 out;                   // [T, n_heads * head_dim]
    const int* cu_q = nullptr;     // [n_seqs + 1] (needed by the query-tile kernel)
    const int* ctx_len = nullptr;  // [n_seqs]
    int max_q_len = 0, max_ctx_len = 0;
    int append = 0;                // != 0: the step's keys/values are still in q's rows: write them to the pages first
    int k_col = 0, v_col = 0;
    const int* slots = nullptr;    // [T] rows of the pages (append)
    int n_single = 0;              // the first n_single sequences bring one token each
    int may_split = 0;             // != 0: the caller takes an AttentionSplits in place of `out`
};

// -- scratch: device memory that kernels need beyond inputs and outputs, one set per stream -----------
// Work on one stream runs in order, so the kernels launched on it can share these buffers; two runners
// (two streams) never share one, so their steps may overlap on the device. A part says what its kernels
// need through the reserve_* calls when its runner is built, so that no step allocates; an op that is
// called with more than was reserved (tests call ops directly) grows the buffer, which synchronises the
// device. release_scratch frees a stream's buffers (the owner of the stream calls it before it destroys it).
void reserve_attention_scratch(int rows, int n_heads, int head_dim, hipStream_t stream);
void reserve_sampling_scratch(int rows, int vocab, hipStream_t stream);
void reserve_linear_scratch(hipStream_t stream);
void release_scratch(hipStream_t stream);
void* scratch_address(const char* name, hipStream_t stream);      // nullptr if not allocated yet (tests)
size_t scratch_bytes();                                            // all streams of the current device (tests)

// -- tuning hooks (tests and tuning scripts) ---------------------------------------------------------
struct Tuning {
    int decode_nsplit = 0, decode_waves = 0;          // > 0: forced launch shape of merged decode attention
    int unmerged_nsplit = 0, unmerged_waves = 0;      // > 0: forced shape of splits merged by the next product
    int merge_max_rows = 16;                          // tokens whose splits a product merges while loading
    int long_context_splits = 1;                      // 1: few pairs with long contexts are split over up to 256 workgroups
    int ln_fuse_max_rows = 32;                        // rows up to which the norm is fused into the few-row product
    // what the ops chose since the last reset (tests read it back instead of trusting the thresholds)
    struct Seen {
        int max_decode_splits = 0;                    // most workgroups a (token, head) pair's keys were split over
        long long merge_kernel_launches = 0, prefill_tile_launches = 0, tiled_f32_launches = 0, generic_attention_launches = 0;
    } seen;
};
Tuning& tuning();

// Token ids that an earlier step sampled on the device and the host has not read yet: where src[t] >= 0,
// token t's id is prev[src[t]] (n_prev entries) and not ids[t].
struct FedTokens {
    const int* src = nullptr;
    const int* prev = nullptr;
    int n_prev = 0;
};

// -- the ops -----------------------------------------------------------------------------------------
void embed(const int* ids, const int* positions, const Tensor2& wte, const Tensor2* wpe, const Tensor2& out,
           hipStream_t stream, const FedTokens* fed = nullptr);
void select_tokens(int* ids, const int* src, const int* prev, int n, int n_prev, hipStream_t stream);
void reset_state(void* state, size_t slot_bytes, int n_slots, const int* slots, const int* starts, int n_seqs,
                 hipStream_t stream);
// out[i,:] = LayerNorm(x[rows ? rows[i] : i, :]); out.rows rows.
void layernorm(const Tensor2& x, const float* gamma, const float* beta, float eps, const Tensor2& out,
               const int* rows, hipStream_t stream);
void kv_append(const Tensor2& src, int k_col, int v_col, const Tensor2& k_pages, const Tensor2& v_pages,
               const int* slots, hipStream_t stream);
// out = epilogue(a w^T + bias); a [M,K], w [N,K] of one dtype, bias fp32 [N] or null.
void linear(const Tensor2& a, const Tensor2& w, const float* bias, const Tensor2& out, int epilogue,
            const KvScatter* kv, hipStream_t stream);
// The same with a = the merged attention splits. `tmp` ([n_tokens, n_heads*head_dim] in w's dtype) is
// used only if the merging kernel does not take these sizes (then: merge kernel, ordinary product).
void linear_from_splits(const AttentionSplits& a, const Tensor2& w, const float* bias, const Tensor2& out,
                        int epilogue, void* tmp, hipStream_t stream);
void merge_splits(const AttentionSplits& a, const Tensor2& out, hipStream_t stream);
// out = epilogue(LayerNorm(x[rows]) w^T + bias), the norm fused into the product where the kernels allow;
// `tmp` ([out.rows, K] in w's dtype) holds the normalised rows otherwise. `kv` as for linear.
void ln_linear(const Tensor2& x, const float* gamma, const float* beta, float eps, const Tensor2& w,
               const float* bias, const Tensor2& out, int epilogue, const int* rows, void* tmp,
               const KvScatter* kv, hipStream_t stream);
// Causal attention of the step's queries over the pages. Returns true and fills *splits when the result is
// left unmerged (only with may_split); otherwise `out` holds it.
bool paged_attention(const AttentionArgs& a, AttentionSplits* splits, hipStream_t stream);
// `mirror` (optional): a second place for the chosen tokens, which may be pinned host memory (the kernel that
// chooses writes it: no copy has to be launched for the host to read them).
void argmax(const Tensor2& logits, int* out, hipStream_t stream, int* mirror = nullptr);
void sample(const Tensor2& logits, const float* temperature, const float* u, int* out, hipStream_t stream, int* mirror = nullptr);

}  // namespace minillm
