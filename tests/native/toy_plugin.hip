// A plugin for the engine, defined entirely under tests/: toy parts and toy architectures that the
// framework's own files know nothing about. Loaded with `--plugin` (command line), MINI_LLM_PLUGINS
// (environment) or mini_llm_amd.load_plugin (Python); its static initialiser registers everything.
//
// Parts (none of them is anyone's model):
//   toy_running_mean  mixer with a fixed-size state of its own per request:
//                     state <- decay * state + (1 - decay) * h_t, token by token; x_t += gain * state
//   toy_scale_norm    norm: x / sqrt(mean(x^2) + eps) * gain
//   toy_identity      norm: the rows, cast to the compute dtype
//   toy_half_turn     position encoding inside the mixer: per head, the pair (v[i], v[i + dh/2]) of
//                     queries and keys is turned by the angle pos * base^(-i / (dh/2))
//   toy_one_of_n      feed-forward with routing: p = softmax(h R^T) in fp32, the token goes to expert
//                     e = argmax p and x += p_e * W2_e gelu(W1_e h)
// Architectures:
//   ToyLM             an attention layer (one key/value head, two norms of different kinds) and a layer
//                     without feed-forward whose mixer is toy_running_mean; the order names the attention
//                     layer twice, the second call only reads the cache the first one wrote; no positions
//   ToyRoutedLM       toy_half_turn, grouped heads, a window in the second layer, toy_one_of_n in the first
//   ToyBareMixer      the attention mixer alone: the embedding table holds the mixer's input rows, norms
//                     are identities, the (untied) head is whatever matrix the checkpoint holds
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>

#include <cmath>

#include "arch.h"

using namespace minillm;

namespace {

// ---------------------------------------------------------------------------------------------
// kernels (plain: these are test parts)
// ---------------------------------------------------------------------------------------------
template <typename T> __device__ inline float to_f(T v);
template <> __device__ inline float to_f<float>(float v) { return v; }
template <> __device__ inline float to_f<__hip_bfloat16>(__hip_bfloat16 v) { return __bfloat162float(v); }
template <typename T> __device__ inline T from_f(float v);
template <> __device__ inline float from_f<float>(float v) { return v; }
template <> __device__ inline __hip_bfloat16 from_f<__hip_bfloat16>(float v) { return __float2bfloat16(v); }

// one workgroup of 64 threads per output row; mode 0: identity, 1: scale norm
template <typename T>
__global__ void toy_norm_kernel(const float* x, const int* rows, const float* gain, T* out, int D, float eps, int mode) {
    const int r = blockIdx.x, src = rows ? rows[r] : r;
    const float* xr = x + static_cast<size_t>(src) * D;
    float scale = 1.f;
    if (mode == 1) {
        float ss = 0.f;
        for (int d = threadIdx.x; d < D; d += 64) ss += xr[d] * xr[d];
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
        scale = 1.f / sqrtf(ss / D + eps);
    }
    for (int d = threadIdx.x; d < D; d += 64)
        out[static_cast<size_t>(r) * D + d] = from_f<T>(mode == 1 ? xr[d] * scale * gain[d] : xr[d]);
}

// one workgroup per sequence, threads over features; the sequence's tokens one after the other
template <typename T>
__global__ void running_mean_kernel(const T* h, const int* cu_q, const int* state_slots, float* state, const float* gain,
                                    float* x, int D, float decay, int write) {
    const int b = blockIdx.x, slot = state_slots[b];
    if (slot < 0) return;                                     // a padding row
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float s = state[static_cast<size_t>(slot) * D + d];
        for (int t = cu_q[b]; t < cu_q[b + 1]; ++t) {
            s = decay * s + (1.f - decay) * to_f<T>(h[static_cast<size_t>(t) * D + d]);
            x[static_cast<size_t>(t) * D + d] += gain[d] * s;
        }
        if (write) state[static_cast<size_t>(slot) * D + d] = s;
    }
}

// one thread per (token, head among queries and keys, pair index)
template <typename T>
__global__ void half_turn_kernel(T* qkv, int stride, const int* positions, int n_tokens, int heads, int head_dim, float base) {
    const int half = head_dim / 2;
    const long long i = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x;
    if (i >= static_cast<long long>(n_tokens) * heads * half) return;
    const int p = static_cast<int>(i % half), hd = static_cast<int>((i / half) % heads), t = static_cast<int>(i / (static_cast<long long>(half) * heads));
    const float angle = static_cast<float>(positions[t]) * powf(base, -static_cast<float>(p) / half);
    const float c = cosf(angle), s = sinf(angle);
    T* v = qkv + static_cast<size_t>(t) * stride + hd * head_dim;
    const float a = to_f<T>(v[p]), b = to_f<T>(v[p + half]);
    v[p] = from_f<T>(a * c - b * s);
    v[p + half] = from_f<T>(b * c + a * s);
}

// one wavefront per token: router logits, the chosen expert and its probability
template <typename T>
__global__ void route_kernel(const T* h, const float* router, int D, int n_experts, float* gate, int* chosen) {
    const int t = blockIdx.x;
    float best = -INFINITY, sum = 0.f;
    int arg = 0;
    float logits[16];
    for (int e = 0; e < n_experts; ++e) {
        float acc = 0.f;
        for (int d = threadIdx.x; d < D; d += 64) acc += to_f<T>(h[static_cast<size_t>(t) * D + d]) * router[static_cast<size_t>(e) * D + d];
        for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
        logits[e] = acc;
        if (acc > best) { best = acc; arg = e; }
    }
    for (int e = 0; e < n_experts; ++e) sum += expf(logits[e] - best);
    if (threadIdx.x == 0) { gate[t] = 1.f / sum; chosen[t] = arg; }
}

__global__ void add_chosen_kernel(float* x, const float* y, const float* gate, const int* chosen, int expert, int T, int D) {
    const long long i = blockIdx.x * static_cast<long long>(blockDim.x) + threadIdx.x;
    if (i >= static_cast<long long>(T) * D) return;
    const int t = static_cast<int>(i / D);
    if (chosen[t] == expert) x[i] += gate[t] * y[i];
}

void launched(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) fail("%s: %s", what, hipGetErrorString(e));
}

const float* f32_vector(const Params& p, const char* key, int n) {
    const Tensor2& t = p.weights(key);
    if (t.dtype != F32 || t.rows * t.cols != n) fail("'%s' must be float32 [%d]", key, n);
    return static_cast<const float*>(t.data);
}

// ---------------------------------------------------------------------------------------------
// parts
// ---------------------------------------------------------------------------------------------
class ToyNorm final : public Norm {
public:
    ToyNorm(const Params& p, int mode) : mode_(mode) {
        size_ = p.integer("size");
        dtype = p.integer("dtype");
        if (mode == 1) { eps_ = static_cast<float>(p.number("eps")); gain_ = f32_vector(p, "gain", size_); }
    }
    Tensor2 forward(const Tensor2& x, const int* rows, int n, Arena& arena, hipStream_t s) const override {
        if (x.dtype != F32 || x.cols != size_ || !x.contiguous()) fail("toy norm: the input must be contiguous float32 [rows, %d]", size_);
        Tensor2 h = arena.tensor(dtype, n, size_);
        if (dtype == F32) toy_norm_kernel<float><<<n, 64, 0, s>>>(static_cast<const float*>(x.data), rows, gain_, static_cast<float*>(h.data), size_, eps_, mode_);
        else toy_norm_kernel<__hip_bfloat16><<<n, 64, 0, s>>>(static_cast<const float*>(x.data), rows, gain_, static_cast<__hip_bfloat16*>(h.data), size_, eps_, mode_);
        launched("toy norm");
        return h;
    }
    size_t workspace_bytes(int rows) const override { return static_cast<size_t>(rows) * size_ * dtype_size(dtype) + 256; }
    void add_cost(StepCost& c) const override { if (mode_ == 1) c.weight_bytes += 4.0 * size_; }

private:
    int size_ = 0, mode_ = 0;
    float eps_ = 0.f;
    const float* gain_ = nullptr;
};

class RunningMean final : public Mixer {
public:
    explicit RunningMean(const Params& p) {
        size_ = p.integer("size");
        decay_ = static_cast<float>(p.number("decay"));
        dtype_ = p.integer("dtype");
        gain_ = f32_vector(p, "gain", size_);
    }
    void forward(NormedInput& h, const StepView& step, const CacheView& cache, const Tensor2& x, bool write, Arena& arena,
                 hipStream_t s) const override {
        if (cache.kind != 2 || cache.slot_bytes != static_cast<size_t>(size_) * 4) fail("toy_running_mean needs a state of %d floats", size_);
        const Tensor2& in = h.tensor(arena, s);
        // a request's slot is empty when it begins: the cache storage clears it, not the mixer
        if (dtype_ == F32)
            running_mean_kernel<float><<<step.n_seqs, 64, 0, s>>>(static_cast<const float*>(in.data), step.cu_q, step.state_slots, static_cast<float*>(cache.state), gain_, static_cast<float*>(x.data), size_, decay_, write ? 1 : 0);
        else
            running_mean_kernel<__hip_bfloat16><<<step.n_seqs, 64, 0, s>>>(static_cast<const __hip_bfloat16*>(in.data), step.cu_q, step.state_slots, static_cast<float*>(cache.state), gain_, static_cast<float*>(x.data), size_, decay_, write ? 1 : 0);
        launched("toy_running_mean");
    }
    size_t workspace_bytes(int) const override { return 256; }
    CacheNeed cache_need() const override {
        CacheNeed n;
        n.kind = 2;
        n.state_bytes = static_cast<size_t>(size_) * 4;
        return n;
    }
    void add_cost(StepCost& c) const override { c.weight_bytes += 4.0 * size_; }

private:
    int size_ = 0, dtype_ = BF16;
    float decay_ = 0.f;
    const float* gain_ = nullptr;
};

class HalfTurn final : public PositionEncoding {
public:
    explicit HalfTurn(const Params& p) : base_(static_cast<float>(p.number("base"))) {}
    bool applies_in_mixer() const override { return true; }
    void in_mixer(const Tensor2& qkv, int n_heads, int n_kv_heads, int head_dim, const StepView& step, hipStream_t s) const override {
        // queries and keys stand side by side at the head of every row: n_heads + n_kv_heads heads to turn
        const int heads = n_heads + n_kv_heads, T = static_cast<int>(qkv.rows);
        const long long n = static_cast<long long>(T) * heads * (head_dim / 2);
        const int blocks = static_cast<int>((n + 255) / 256);
        if (qkv.dtype == F32) half_turn_kernel<float><<<blocks, 256, 0, s>>>(static_cast<float*>(qkv.data), static_cast<int>(qkv.stride), step.positions, T, heads, head_dim, base_);
        else half_turn_kernel<__hip_bfloat16><<<blocks, 256, 0, s>>>(static_cast<__hip_bfloat16*>(qkv.data), static_cast<int>(qkv.stride), step.positions, T, heads, head_dim, base_);
        launched("toy_half_turn");
    }

private:
    float base_;
};

class OneOfN final : public FeedForward {
public:
    explicit OneOfN(const Params& p) {
        size_ = p.integer("size");
        n_ = p.integer("n_experts");
        dtype_ = p.integer("dtype");
        if (n_ < 1 || n_ > 16) fail("toy_one_of_n: 1 to 16 experts");
        const Tensor2& r = p.weights("router");
        if (r.dtype != F32 || r.rows != n_ || r.cols != size_) fail("toy_one_of_n: the router must be float32 [%d, %d]", n_, size_);
        router_ = static_cast<const float*>(r.data);
        for (int e = 0; e < n_; ++e) {
            up_.emplace_back(p.weights("expert." + std::to_string(e) + ".up"), nullptr);
            down_.emplace_back(p.weights("expert." + std::to_string(e) + ".down"), nullptr);
        }
        inner_ = up_[0].out_features();
    }
    void forward(NormedInput& h, const StepView& step, const Tensor2& x, Arena& arena, hipStream_t s) const override {
        const int T = step.n_tokens;
        const Tensor2& in = h.tensor(arena, s);
        float* gate = static_cast<float*>(arena.take(static_cast<size_t>(T) * 4));
        int* chosen = static_cast<int*>(arena.take(static_cast<size_t>(T) * 4));
        if (dtype_ == F32) route_kernel<float><<<T, 64, 0, s>>>(static_cast<const float*>(in.data), router_, size_, n_, gate, chosen);
        else route_kernel<__hip_bfloat16><<<T, 64, 0, s>>>(static_cast<const __hip_bfloat16*>(in.data), router_, size_, n_, gate, chosen);
        launched("toy_one_of_n (routing)");
        Tensor2 inner = arena.tensor(dtype_, T, inner_), y = arena.tensor(F32, T, size_);
        // every expert runs on every token through the engine's own products; only the chosen one's output is added
        for (int e = 0; e < n_; ++e) {
            up_[e](in, inner, GELU_ERF, nullptr, s);
            down_[e](inner, y, STORE_F32, nullptr, s);
            const long long n = static_cast<long long>(T) * size_;
            add_chosen_kernel<<<static_cast<int>((n + 255) / 256), 256, 0, s>>>(static_cast<float*>(x.data), static_cast<const float*>(y.data), gate, chosen, e, T, size_);
            launched("toy_one_of_n (add)");
        }
    }
    size_t workspace_bytes(int tokens) const override {
        return static_cast<size_t>(tokens) * (8 + inner_ * dtype_size(dtype_) + size_ * 4) + 2048;
    }
    void reserve(int, hipStream_t s) const override { reserve_linear_scratch(s); }
    void add_cost(StepCost& c) const override {
        for (int e = 0; e < n_; ++e) { up_[e].add_cost(c); down_[e].add_cost(c); }
        c.weight_bytes += 4.0 * n_ * size_;
    }

private:
    int size_ = 0, inner_ = 0, n_ = 0, dtype_ = BF16;
    const float* router_ = nullptr;
    std::vector<Linear> up_, down_;
};

// ---------------------------------------------------------------------------------------------
// architectures
// ---------------------------------------------------------------------------------------------
int64_t need_int(const Json& c, const char* key) {
    const Json* v = c.find(key);
    if (v == nullptr || !v->is_integer()) throw ConfigError(std::string("config.json: integer key '") + key + "' is missing");
    if (v->integer() <= 0) throw ConfigError(std::string("config.json: '") + key + "' must be positive");
    return v->integer();
}
double need_num(const Json& c, const char* key) {
    const Json* v = c.find(key);
    if (v == nullptr || !v->is_number()) throw ConfigError(std::string("config.json: number key '") + key + "' is missing");
    return v->number();
}

struct Specs {
    std::vector<ParamSpec> s;
    void matrix(const std::string& n, int64_t r, int64_t k, double std = 0.02) { s.push_back({n, {r, k}, ParamSpec::Matrix, false, 0.0, std}); }
    void vector(const std::string& n, int64_t k, double mean, double std) { s.push_back({n, {k}, ParamSpec::Vector, false, mean, std}); }
    void table(const std::string& n, int64_t r, int64_t k, double std) { s.push_back({n, {r, k}, ParamSpec::Vector, false, 0.0, std}); }   // kept in fp32
};

std::unique_ptr<Norm> layer_norm(const std::map<std::string, Tensor2>& t, const std::string& name, int64_t size, double eps, int dtype) {
    Params p;
    p.num["size"] = static_cast<double>(size); p.num["eps"] = eps; p.num["dtype"] = dtype;
    p.tensor["gamma"] = t.at(name + ".weight");
    p.tensor["beta"] = t.at(name + ".bias");
    return build_norm("layernorm", p);
}

Params attention_params(const std::map<std::string, Tensor2>& t, const std::string& pre, int heads, int kv_heads, int head_dim, int window,
                        bool bias, int dtype) {
    Params a;
    a.num["n_heads"] = heads; a.num["n_kv_heads"] = kv_heads; a.num["head_dim"] = head_dim;
    a.num["scale"] = 1.0 / std::sqrt(static_cast<double>(head_dim));
    a.num["window"] = window; a.num["dtype"] = dtype;
    a.tensor["qkv.weight"] = t.at(pre + "qkv.weight");
    a.tensor["out.weight"] = t.at(pre + "o.weight");
    if (bias) { a.tensor["qkv.bias"] = t.at(pre + "qkv.bias"); a.tensor["out.bias"] = t.at(pre + "o.bias"); }
    return a;
}

void embedding_and_tied_head(const std::map<std::string, Tensor2>& t, int dtype, DecoderModel& m) {
    Params e, h;
    e.tensor["table"] = t.at("emb.weight");
    m.embedding = build_embedding("token_table", e);
    h.tensor["weight"] = t.at("emb.weight");
    h.num["dtype"] = dtype;
    m.head = build_head("linear", h);
}

// -- ToyLM --------------------------------------------------------------------------------------------
std::vector<ParamSpec> toy_specs(const Json& c) {
    const int64_t V = need_int(c, "vocab"), D = need_int(c, "width"), H = need_int(c, "heads");
    if (D % H != 0) throw ConfigError("config.json: width is not divisible by heads");
    const int64_t dh = D / H;
    Specs s;
    s.matrix("emb.weight", V, D);
    s.vector("l0.n1.weight", D, 1.0, 0.1); s.vector("l0.n1.bias", D, 0.0, 0.02);
    s.matrix("l0.qkv.weight", D + 2 * dh, D); s.matrix("l0.o.weight", D, D);
    s.vector("l0.n2.gain", D, 1.0, 0.1);
    s.matrix("l0.up.weight", 2 * D, D); s.matrix("l0.down.weight", D, 2 * D);
    s.vector("l1.n1.weight", D, 1.0, 0.1); s.vector("l1.n1.bias", D, 0.0, 0.02);
    s.vector("l1.mean.gain", D, 1.0, 0.1);
    s.vector("final.weight", D, 1.0, 0.1); s.vector("final.bias", D, 0.0, 0.02);
    return s.s;
}

void toy_assemble(const Json& c, const std::map<std::string, Tensor2>& t, int dtype, LoadedModel& out) {
    const int D = static_cast<int>(need_int(c, "width")), H = static_cast<int>(need_int(c, "heads"));
    const double eps = need_num(c, "eps"), decay = need_num(c, "decay");
    DecoderModel& m = out.model;
    embedding_and_tied_head(t, dtype, m);                   // no position encoding at all
    {
        // layer 0: attention with one key/value head, then a feed-forward behind a norm of another kind
        Params f, n2;
        f.str["activation"] = "gelu_erf"; f.num["dtype"] = dtype;
        f.tensor["up.weight"] = t.at("l0.up.weight"); f.tensor["down.weight"] = t.at("l0.down.weight");
        n2.num["size"] = D; n2.num["eps"] = 10 * eps; n2.num["dtype"] = dtype; n2.tensor["gain"] = t.at("l0.n2.gain");
        std::vector<std::unique_ptr<Norm>> norms;
        norms.push_back(layer_norm(t, "l0.n1", D, eps, dtype));
        norms.push_back(build_norm("toy_scale_norm", n2));
        m.layers.push_back(build_block("pre_norm", build_mixer("causal_attention", attention_params(t, "l0.", H, 1, D / H, 0, false, dtype)),
                                       build_feed_forward("dense_mlp", f), std::move(norms)));
    }
    {
        // layer 1: the stateful mixer, no feed-forward
        Params r;
        r.num["size"] = D; r.num["decay"] = decay; r.num["dtype"] = dtype; r.tensor["gain"] = t.at("l1.mean.gain");
        std::vector<std::unique_ptr<Norm>> norms;
        norms.push_back(layer_norm(t, "l1.n1", D, eps, dtype));
        m.layers.push_back(build_block("pre_norm", build_mixer("toy_running_mean", r), nullptr, std::move(norms)));
    }
    // the attention layer runs twice; its second call only reads the cache that the first one wrote
    m.order = {{0, 0, true}, {1, 1, true}, {0, 0, false}};
    m.final_norm = layer_norm(t, "final", D, eps, dtype);
    if (const Json* e = c.find("eos")) if (e->is_integer()) out.eos_token_id = static_cast<int>(e->integer());
}

// -- ToyRoutedLM --------------------------------------------------------------------------------------
std::vector<ParamSpec> routed_specs(const Json& c) {
    const int64_t V = need_int(c, "vocab"), D = need_int(c, "width"), H = need_int(c, "heads"), G = need_int(c, "groups"),
                  E = need_int(c, "experts");
    if (D % H != 0 || H % G != 0) throw ConfigError("config.json: width / heads / groups do not divide");
    const int64_t dh = D / H;
    Specs s;
    s.matrix("emb.weight", V, D);
    for (int l = 0; l < 2; ++l) {
        const std::string p = "l" + std::to_string(l) + ".";
        s.vector(p + "n1.weight", D, 1.0, 0.1); s.vector(p + "n1.bias", D, 0.0, 0.02);
        s.matrix(p + "qkv.weight", D + 2 * G * dh, D); s.vector(p + "qkv.bias", D + 2 * G * dh, 0.0, 0.02);
        s.matrix(p + "o.weight", D, D); s.vector(p + "o.bias", D, 0.0, 0.02);
        s.vector(p + "n2.weight", D, 1.0, 0.1); s.vector(p + "n2.bias", D, 0.0, 0.02);
    }
    s.table("l0.router", E, D, 1.0);
    for (int64_t e = 0; e < E; ++e) {
        s.matrix("l0.expert." + std::to_string(e) + ".up", 2 * D, D);
        s.matrix("l0.expert." + std::to_string(e) + ".down", D, 2 * D);
    }
    s.matrix("l1.up.weight", 3 * D, D); s.vector("l1.up.bias", 3 * D, 0.0, 0.02);
    s.matrix("l1.down.weight", D, 3 * D); s.vector("l1.down.bias", D, 0.0, 0.02);
    s.vector("final.weight", D, 1.0, 0.1); s.vector("final.bias", D, 0.0, 0.02);
    return s.s;
}

void routed_assemble(const Json& c, const std::map<std::string, Tensor2>& t, int dtype, LoadedModel& out) {
    const int D = static_cast<int>(need_int(c, "width")), H = static_cast<int>(need_int(c, "heads")), G = static_cast<int>(need_int(c, "groups")),
              E = static_cast<int>(need_int(c, "experts")), W = static_cast<int>(need_int(c, "window"));
    const double eps = need_num(c, "eps");
    DecoderModel& m = out.model;
    embedding_and_tied_head(t, dtype, m);
    Params turn;
    turn.num["base"] = need_num(c, "base");
    m.position = build_position("toy_half_turn", turn);
    for (int l = 0; l < 2; ++l) {
        const std::string p = "l" + std::to_string(l) + ".";
        Params a = attention_params(t, p, H, G, D / H, l == 1 ? W : 0, true, dtype);
        a.position = m.position;                            // the mixer turns its queries and keys with it
        std::unique_ptr<FeedForward> ff;
        if (l == 0) {
            Params r;
            r.num["size"] = D; r.num["n_experts"] = E; r.num["dtype"] = dtype;
            r.tensor["router"] = t.at("l0.router");
            for (int e = 0; e < E; ++e) {
                r.tensor["expert." + std::to_string(e) + ".up"] = t.at("l0.expert." + std::to_string(e) + ".up");
                r.tensor["expert." + std::to_string(e) + ".down"] = t.at("l0.expert." + std::to_string(e) + ".down");
            }
            ff = build_feed_forward("toy_one_of_n", r);
        } else {
            Params f;
            f.str["activation"] = "gelu_tanh"; f.num["dtype"] = dtype;
            f.tensor["up.weight"] = t.at("l1.up.weight"); f.tensor["up.bias"] = t.at("l1.up.bias");
            f.tensor["down.weight"] = t.at("l1.down.weight"); f.tensor["down.bias"] = t.at("l1.down.bias");
            ff = build_feed_forward("dense_mlp", f);
        }
        std::vector<std::unique_ptr<Norm>> norms;
        norms.push_back(layer_norm(t, p + "n1", D, eps, dtype));
        norms.push_back(layer_norm(t, p + "n2", D, eps, dtype));
        m.layers.push_back(build_block("pre_norm", build_mixer("causal_attention", a), std::move(ff), std::move(norms)));
        m.order.push_back({l, l, true});
    }
    m.final_norm = layer_norm(t, "final", D, eps, dtype);
}

// -- ToyBareMixer -------------------------------------------------------------------------------------
std::vector<ParamSpec> bare_specs(const Json& c) {
    const int64_t R = need_int(c, "rows"), H = need_int(c, "heads"), G = need_int(c, "kv_heads"), dh = need_int(c, "head_dim"),
                  O = need_int(c, "outputs");
    const int64_t D = H * dh;
    const bool bias = c.find("bias") != nullptr && c.at("bias").is_bool() && c.at("bias").boolean();
    Specs s;
    s.matrix("emb.weight", R, D, 1.0);
    s.matrix("qkv.weight", D + 2 * G * dh, D, 0.2); s.matrix("o.weight", D, D, 0.2);
    if (bias) { s.vector("qkv.bias", D + 2 * G * dh, 0.0, 0.2); s.vector("o.bias", D, 0.0, 0.2); }
    s.matrix("head.weight", O, D, 1.0);
    return s.s;
}

void bare_assemble(const Json& c, const std::map<std::string, Tensor2>& t, int dtype, LoadedModel& out) {
    const int H = static_cast<int>(need_int(c, "heads")), G = static_cast<int>(need_int(c, "kv_heads")), dh = static_cast<int>(need_int(c, "head_dim"));
    const int D = H * dh;
    const bool bias = c.find("bias") != nullptr && c.at("bias").is_bool() && c.at("bias").boolean();
    const Json* w = c.find("window");
    DecoderModel& m = out.model;
    Params e, h, id;
    e.tensor["table"] = t.at("emb.weight");
    m.embedding = build_embedding("token_table", e);
    h.tensor["weight"] = t.at("head.weight");               // an untied head
    h.num["dtype"] = dtype;
    m.head = build_head("linear", h);
    id.num["size"] = D; id.num["dtype"] = dtype;
    std::vector<std::unique_ptr<Norm>> norms;
    norms.push_back(build_norm("toy_identity", id));
    m.layers.push_back(build_block("pre_norm", build_mixer("causal_attention", attention_params(t, "", H, G, dh, (w && w->is_integer()) ? static_cast<int>(w->integer()) : 0, bias, dtype)),
                                   nullptr, std::move(norms)));
    m.order = {{0, 0, true}};
    m.final_norm = build_norm("toy_identity", id);
}

struct Registration {
    Registration() {
        register_norm("toy_scale_norm", [](const Params& p) { return std::unique_ptr<Norm>(new ToyNorm(p, 1)); });
        register_norm("toy_identity", [](const Params& p) { return std::unique_ptr<Norm>(new ToyNorm(p, 0)); });
        register_mixer("toy_running_mean", [](const Params& p) { return std::unique_ptr<Mixer>(new RunningMean(p)); });
        register_position("toy_half_turn", [](const Params& p) { return std::shared_ptr<const PositionEncoding>(new HalfTurn(p)); });
        register_feed_forward("toy_one_of_n", [](const Params& p) { return std::unique_ptr<FeedForward>(new OneOfN(p)); });
        Architecture a;
        a.name = "ToyLM"; a.param_specs = toy_specs; a.assemble = toy_assemble;
        register_architecture(a);
        a.name = "ToyRoutedLM"; a.param_specs = routed_specs; a.assemble = routed_assemble;
        register_architecture(a);
        a.name = "ToyBareMixer"; a.param_specs = bare_specs; a.assemble = bare_assemble;
        register_architecture(a);
    }
} registration;

}  // namespace
