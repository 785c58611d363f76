// Plain C++ twins of the device operations, one per kernel: whole loops on the CPU, float32 inputs,
// sums in double, no tiling, no paging tricks. They are the oracle that the kernel tests compare with
// (beside the plain Python references), and what a reader checks a kernel's meaning against. They
// share no code with the kernels or the engine.
//
// The reference keeps a CPU check beside its kernels in its tests
// (/root/reference/tests/cpp/test_flashattention.cu:39-105 naive attention in double,
//  /root/reference/tests/cpp/test_gemm.cu:316-348 reference_linear).
#include <cmath>
#include <cstdint>
#include <limits>
#include <vector>

extern "C" {

// x[t,:] = wte[ids[t],:] + wpe[pos[t],:]   -- /root/reference/src/kernels/embedding.cu:23-43
void ref_embed(const int* ids, const int* pos, const float* wte, const float* wpe, float* out, int T, int D) {
    for (int t = 0; t < T; ++t)
        for (int d = 0; d < D; ++d)
            out[static_cast<size_t>(t) * D + d] =
                wte[static_cast<size_t>(ids[t]) * D + d] + (wpe ? wpe[static_cast<size_t>(pos[t]) * D + d] : 0.f);
}

// mean; biased variance of (x - mean); (x - mean) / sqrt(var + eps) * gamma + beta
// -- /root/reference/src/kernels/layernorm.cu:32-49. rows (optional) selects input rows.
void ref_layernorm(const float* x, const int* rows, const float* gamma, const float* beta, float eps, float* out, int n,
                   int D) {
    for (int r = 0; r < n; ++r) {
        const float* xr = x + static_cast<size_t>(rows ? rows[r] : r) * D;
        double mean = 0.0;
        for (int d = 0; d < D; ++d) mean += xr[d];
        mean /= D;
        double var = 0.0;
        for (int d = 0; d < D; ++d) var += (xr[d] - mean) * (xr[d] - mean);
        var /= D;
        const double inv = 1.0 / std::sqrt(var + static_cast<double>(eps));
        for (int d = 0; d < D; ++d)
            out[static_cast<size_t>(r) * D + d] = static_cast<float>((xr[d] - mean) * inv * gamma[d] + (beta ? beta[d] : 0.f));
    }
}

// 0.5 v (1 + tanh(0.7978845608 (v + 0.044715 v^3)))  -- /root/reference/src/kernels/gelu.cu:7-9
static double gelu_tanh(double v) { return 0.5 * v * (1.0 + std::tanh(0.7978845608 * (v + 0.044715 * v * v * v))); }
// 0.5 v (1 + erf(v / sqrt 2)): the exact form (the reference has only the tanh form)
static double gelu_erf(double v) { return 0.5 * v * (1.0 + std::erf(v * 0.70710678118654752440)); }

// The epilogues as operations of their own (the reference: /root/reference/src/kernels/gelu.cu:7-21,
// /root/reference/src/kernels/residual.cu:6-31; its bias is added inside the product, linear.cu:8-27).
void ref_gelu(const float* x, float* out, long n, int exact) {
    for (long i = 0; i < n; ++i) out[i] = static_cast<float>(exact ? gelu_erf(x[i]) : gelu_tanh(x[i]));
}
void ref_add_bias(float* x, const float* bias, int M, int N) {
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) x[static_cast<size_t>(m) * N + n] += bias[n];
}
void ref_residual_add(float* x, const float* y, long n) {
    for (long i = 0; i < n; ++i) x[i] += y[i];
}

// out = epilogue(a w^T + bias): a [M,K], w [N,K] (both k-contiguous), bias [N] or null.
// epilogue: 0 store, 1 gelu_tanh, 2 gelu_erf, 3 add into out, 4 store (the kernels' fp32 store)
// -- /root/reference/src/kernels/linear.cu:8-87, the store path /root/reference/src/kernels/gemm.cu:534-564
int ref_linear(const float* a, const float* w, const float* bias, float* out, int M, int N, int K, int epilogue) {
    if (epilogue < 0 || epilogue > 4) return -1;
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int k = 0; k < K; ++k) acc += static_cast<double>(a[static_cast<size_t>(m) * K + k]) * w[static_cast<size_t>(n) * K + k];
            if (bias) acc += bias[n];
            float* o = out + static_cast<size_t>(m) * N + n;
            if (epilogue == 1) acc = gelu_tanh(acc);
            if (epilogue == 2) acc = gelu_erf(acc);
            *o = static_cast<float>(epilogue == 3 ? *o + acc : acc);
        }
    return 0;
}

// Key and value columns of each row to row slots[t] of the pages (slot < 0: skipped)
// -- /root/reference/src/kernels/prefill/append_kv.cu:28-46
void ref_kv_append(const float* src, int src_stride, int k_col, int v_col, float* k_pages, float* v_pages, int kv_dim,
                   const int* slots, int T) {
    for (int t = 0; t < T; ++t) {
        if (slots[t] < 0) continue;
        for (int d = 0; d < kv_dim; ++d) {
            k_pages[static_cast<size_t>(slots[t]) * kv_dim + d] = src[static_cast<size_t>(t) * src_stride + k_col + d];
            v_pages[static_cast<size_t>(slots[t]) * kv_dim + d] = src[static_cast<size_t>(t) * src_stride + v_col + d];
        }
    }
}

// Causal attention of every token over its sequence's keys in the pages: for the query at position p of
// head h, s_j = (q_h . k_{j,h}) * scale for keys j in [max(0, p - window + 1) if window else 0, p],
// softmax with the maximum subtracted, o_h = sum_j w_j v_{j,h}; no 1e-6 in the denominator.
// -- /root/reference/src/kernels/prefill/flashattention.cu:71-79,129-178,
//    /root/reference/src/kernels/decode/paged_attention.cu:58-120 (its three passes)
void ref_paged_attention(const float* q, int q_stride, int q_col, int n_heads, int n_kv_heads, int head_dim,
                         const float* k_pages, const float* v_pages, int page_size, const int* block_tables,
                         int max_blocks, const int* token_seq, const int* positions, float scale, int window, float* out,
                         int T) {
    const int kv_dim = n_kv_heads * head_dim, rep = n_heads / n_kv_heads;
    std::vector<double> s;
    for (int t = 0; t < T; ++t) {
        const int b = token_seq[t], p = positions[t];
        const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
        for (int h = 0; h < n_heads; ++h) {
            const int hk = h / rep;
            const float* qh = q + static_cast<size_t>(t) * q_stride + q_col + h * head_dim;
            s.assign(p - lo + 1, 0.0);
            double mx = -std::numeric_limits<double>::infinity();
            for (int j = lo; j <= p; ++j) {
                const size_t row = static_cast<size_t>(block_tables[static_cast<size_t>(b) * max_blocks + j / page_size]) * page_size + j % page_size;
                double d = 0.0;
                for (int e = 0; e < head_dim; ++e) d += static_cast<double>(qh[e]) * k_pages[row * kv_dim + hk * head_dim + e];
                s[j - lo] = d * scale;
                mx = std::max(mx, s[j - lo]);
            }
            double sum = 0.0;
            for (double& v : s) { v = std::exp(v - mx); sum += v; }
            for (int e = 0; e < head_dim; ++e) {
                double o = 0.0;
                for (int j = lo; j <= p; ++j) {
                    const size_t row = static_cast<size_t>(block_tables[static_cast<size_t>(b) * max_blocks + j / page_size]) * page_size + j % page_size;
                    o += s[j - lo] * v_pages[row * kv_dim + hk * head_dim + e];
                }
                out[static_cast<size_t>(t) * n_heads * head_dim + h * head_dim + e] = static_cast<float>(o / sum);
            }
        }
    }
}

// Index of the largest value of each row, the lowest index on ties -- /root/reference/src/kernels/argmax.cu:12-20
void ref_argmax(const float* logits, int n, int V, int* out) {
    for (int r = 0; r < n; ++r) {
        int best = 0;
        for (int i = 1; i < V; ++i)
            if (logits[static_cast<size_t>(r) * V + i] > logits[static_cast<size_t>(r) * V + best]) best = i;
        out[r] = best;
    }
}

// temperature <= 0: argmax. Otherwise the first index whose cumulative mass of exp((l - max) / temperature)
// exceeds u * total (inverse CDF; the reference samples greedily only).
void ref_sample(const float* logits, int n, int V, const float* temperature, const float* u, int* out) {
    for (int r = 0; r < n; ++r) {
        const float* row = logits + static_cast<size_t>(r) * V;
        int best = 0;
        for (int i = 1; i < V; ++i)
            if (row[i] > row[best]) best = i;
        out[r] = best;
        if (temperature[r] <= 0.f) continue;
        double total = 0.0;
        for (int i = 0; i < V; ++i) total += std::exp((static_cast<double>(row[i]) - row[best]) / temperature[r]);
        const double target = static_cast<double>(u[r]) * total;
        double c = 0.0;
        int pick = V - 1;
        for (int i = 0; i < V; ++i) {
            c += std::exp((static_cast<double>(row[i]) - row[best]) / temperature[r]);
            if (c > target) { pick = i; break; }
        }
        out[r] = pick;
    }
}

}  // extern "C"
