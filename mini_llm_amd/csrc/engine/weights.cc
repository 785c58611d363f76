#include "weights.h"

#include <fcntl.h>
#include <hip/hip_runtime.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cmath>
#include <cstring>
#include <fstream>
#include <functional>
#include <set>
#include <sstream>
#include <thread>

namespace minillm {

// ---------------------------------------------------------------------------------------------
// safetensors
// ---------------------------------------------------------------------------------------------
static size_t dtype_bytes(const std::string& dt, const std::string& path, const std::string& name) {
    if (dt == "F32" || dt == "I32") return 4;
    if (dt == "BF16" || dt == "F16") return 2;
    if (dt == "F64" || dt == "I64") return 8;
    if (dt == "U8" || dt == "BOOL" || dt == "I8") return 1;
    throw WeightsError(path + ": tensor '" + name + "' has unsupported dtype " + dt);
}

SafetensorsFile::SafetensorsFile(const std::string& path) : path_(path) {
    const int fd = ::open(path.c_str(), O_RDONLY);
    if (fd < 0) throw WeightsError(path + ": cannot be opened");
    struct stat st;
    if (fstat(fd, &st) != 0) { ::close(fd); throw WeightsError(path + ": cannot be examined"); }
    size_ = static_cast<size_t>(st.st_size);
    if (size_ < 8) { ::close(fd); throw WeightsError(path + ": too short to be a safetensors file (" + std::to_string(size_) + " bytes)"); }
    map_ = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd, 0);
    ::close(fd);
    if (map_ == MAP_FAILED) { map_ = nullptr; throw WeightsError(path + ": cannot be mapped"); }
    const unsigned char* base = static_cast<const unsigned char*>(map_);
    uint64_t hlen = 0;
    for (int i = 7; i >= 0; --i) hlen = (hlen << 8) | base[i];
    // (compared without adding to hlen, which may be anything up to 2^64 - 1; headers beyond 100 MB are refused
    // as the format's own library does)
    if (hlen == 0 || hlen > size_ - 8)
        throw WeightsError(path + ": header length " + std::to_string(hlen) + " exceeds the file size " + std::to_string(size_));
    if (hlen > 100u * 1000u * 1000u) throw WeightsError(path + ": header of " + std::to_string(hlen) + " bytes is larger than 100 MB");
    Json header;
    try {
        header = Json::parse(std::string(reinterpret_cast<const char*>(base + 8), hlen));
    } catch (const JsonError& e) {
        throw WeightsError(path + ": header is not valid JSON (" + e.what() + ")");
    }
    if (!header.is_object()) throw WeightsError(path + ": header is not a JSON object");
    const size_t data_start = 8 + hlen, data_len = size_ - data_start;
    for (const auto& kv : header.members()) {
        if (kv.first == "__metadata__") continue;
        StoredTensor t;
        try {
            t.dtype = kv.second.at("dtype").string();
            for (const Json& s : kv.second.at("shape").array()) t.shape.push_back(s.integer());
            const auto& off = kv.second.at("data_offsets").array();
            if (off.size() != 2) throw JsonError("data_offsets must have two entries");
            const int64_t b = off[0].integer(), e = off[1].integer();
            const int64_t numel = t.numel();
            const size_t esz = dtype_bytes(t.dtype, path, kv.first);
            if (numel < 0 || static_cast<uint64_t>(numel) > UINT64_MAX / 8)
                throw WeightsError(path + ": tensor '" + kv.first + "' has a negative dimension or more elements than can be counted");
            const size_t want = static_cast<size_t>(numel) * esz;
            if (b < 0 || e < b || static_cast<size_t>(e) > data_len)
                throw WeightsError(path + ": tensor '" + kv.first + "' has offsets [" + std::to_string(b) + ", " + std::to_string(e) +
                                   ") outside the file's " + std::to_string(data_len) + " data bytes");
            if (static_cast<size_t>(e - b) != want)
                throw WeightsError(path + ": tensor '" + kv.first + "' holds " + std::to_string(e - b) + " bytes, its shape and dtype need " +
                                   std::to_string(want));
            t.data = base + data_start + b;
            t.bytes = static_cast<size_t>(e - b);
        } catch (const JsonError& e) {
            throw WeightsError(path + ": entry of tensor '" + kv.first + "' is malformed (" + e.what() + ")");
        }
        tensors_.emplace(kv.first, std::move(t));
    }
}

SafetensorsFile::~SafetensorsFile() {
    if (map_ != nullptr) munmap(map_, size_);
}

void save_safetensors(const std::string& path, const std::map<std::string, TensorToStore>& tensors,
                      const std::map<std::string, std::string>& metadata) {
    Json header = Json::object();
    if (!metadata.empty()) {
        Json m = Json::object();
        for (const auto& kv : metadata) m.set(kv.first, Json::of(kv.second));
        header.set("__metadata__", m);
    }
    int64_t off = 0;
    for (const auto& kv : tensors) {       // std::map: sorted names
        Json e = Json::object();
        e.set("dtype", Json::of(kv.second.dtype));
        std::vector<Json> shape;
        for (int64_t s : kv.second.shape) shape.push_back(Json::of(s));
        e.set("shape", Json::array_of(shape));
        const int64_t n = static_cast<int64_t>(kv.second.bytes.size());
        e.set("data_offsets", Json::array_of({Json::of(off), Json::of(off + n)}));
        off += n;
        header.set(kv.first, e);
    }
    std::string h = header.dump();
    while (h.size() % 8 != 0) h += ' ';
    std::ofstream f(path, std::ios::binary);
    if (!f) throw WeightsError(path + ": cannot be written");
    uint64_t hlen = h.size();
    unsigned char len[8];
    for (int i = 0; i < 8; ++i) len[i] = static_cast<unsigned char>(hlen >> (8 * i));
    f.write(reinterpret_cast<const char*>(len), 8);
    f.write(h.data(), static_cast<std::streamsize>(h.size()));
    for (const auto& kv : tensors) f.write(reinterpret_cast<const char*>(kv.second.bytes.data()), static_cast<std::streamsize>(kv.second.bytes.size()));
    if (!f) throw WeightsError(path + ": write failed");
}

// ---------------------------------------------------------------------------------------------
// numbers
// ---------------------------------------------------------------------------------------------
uint64_t splitmix64(uint64_t x) {
    uint64_t z = x + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

uint64_t fnv1a64(const std::string& s) {
    uint64_t h = 0xCBF29CE484222325ull;
    for (const unsigned char c : s) h = (h ^ c) * 0x100000001B3ull;
    return h;
}

void normal_values(uint64_t seed, const std::string& name, int64_t first, int64_t n, double mean, double std,
                   float* out) {
    const uint64_t key = splitmix64(seed) ^ fnv1a64(name);
    const double inv = 1.0 / 9007199254740992.0;
    const double two_pi = 6.283185307179586476925286766559;
    auto piece = [&](int64_t lo, int64_t hi) {
        for (int64_t k = lo; k < hi; ++k) {
            const uint64_t i = static_cast<uint64_t>(first + k);
            const uint64_t a = splitmix64(key + 2 * i), b = splitmix64(key + 2 * i + 1);
            const double u1 = (static_cast<double>(a >> 11) + 1.0) * inv, u2 = static_cast<double>(b >> 11) * inv;
            out[k] = static_cast<float>(mean + std * (std::sqrt(-2.0 * std::log(u1)) * std::cos(two_pi * u2)));
        }
    };
    const int workers = n > (1 << 18) ? static_cast<int>(std::min<unsigned>(16, std::max(1u, std::thread::hardware_concurrency()))) : 1;
    if (workers <= 1) { piece(0, n); return; }
    std::vector<std::thread> pool;
    const int64_t per = (n + workers - 1) / workers;
    for (int w = 0; w < workers; ++w) {
        const int64_t lo = w * per, hi = std::min<int64_t>(n, lo + per);
        if (lo < hi) pool.emplace_back(piece, lo, hi);
    }
    for (auto& t : pool) t.join();
}

uint16_t float_to_bf16_bits(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu)) return static_cast<uint16_t>((u >> 16) | 0x40);   // NaN
    const uint32_t round = 0x7FFFu + ((u >> 16) & 1u);
    return static_cast<uint16_t>((u + round) >> 16);
}

float bf16_bits_to_float(uint16_t b) {
    const uint32_t u = static_cast<uint32_t>(b) << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

float f16_bits_to_float(uint16_t h) {
    const uint32_t sign = (h >> 15) & 1u, exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    float v;
    if (exp == 0) v = std::ldexp(static_cast<float>(man), -24);
    else if (exp == 31) v = man ? NAN : INFINITY;
    else v = std::ldexp(static_cast<float>(man | 0x400u), static_cast<int>(exp) - 25);
    return sign ? -v : v;
}

// ---------------------------------------------------------------------------------------------
// sources
// ---------------------------------------------------------------------------------------------
static bool file_exists(const std::string& p) {
    struct stat st;
    return stat(p.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}

static std::string read_text(const std::string& path) {
    std::ifstream f(path);
    if (!f) throw WeightsError(path + ": cannot be read");
    std::stringstream ss;
    ss << f.rdbuf();
    return ss.str();
}

CheckpointSource::CheckpointSource(const std::string& model_dir) : dir_(model_dir) {
    const std::string single = model_dir + "/model.safetensors", index = model_dir + "/model.safetensors.index.json";
    std::vector<std::string> paths;
    if (file_exists(single)) {
        paths.push_back(single);
    } else if (file_exists(index)) {
        std::set<std::string> shards;
        try {
            const Json j = Json::parse(read_text(index));
            for (const auto& kv : j.at("weight_map").members()) shards.insert(kv.second.string());
        } catch (const JsonError& e) {
            throw WeightsError(index + ": " + e.what());
        }
        for (const auto& s : shards) paths.push_back(model_dir + "/" + s);
    } else {
        throw WeightsError(model_dir + ": neither model.safetensors nor model.safetensors.index.json is there");
    }
    for (const auto& p : paths) {
        files_.emplace_back(new SafetensorsFile(p));
        for (const auto& kv : files_.back()->tensors()) {
            if (all_.count(kv.first)) throw WeightsError(model_dir + ": tensor '" + kv.first + "' appears in two files");
            all_[kv.first] = &kv.second;
        }
    }
}

std::vector<std::string> CheckpointSource::names() const {
    std::vector<std::string> n;
    for (const auto& kv : all_) n.push_back(kv.first);
    return n;
}

const std::vector<int64_t>* CheckpointSource::shape_of(const std::string& name) const {
    auto it = all_.find(name);
    return it == all_.end() ? nullptr : &it->second->shape;
}

void CheckpointSource::read(const ParamSpec& spec, const std::string& stored_name, std::vector<float>& out) const {
    const StoredTensor& t = *all_.at(stored_name);
    const int64_t n = t.numel();
    out.resize(static_cast<size_t>(n));
    if (t.dtype == "F32") {
        std::memcpy(out.data(), t.data, static_cast<size_t>(n) * 4);
    } else if (t.dtype == "BF16") {
        const uint16_t* p = reinterpret_cast<const uint16_t*>(t.data);
        for (int64_t i = 0; i < n; ++i) out[i] = bf16_bits_to_float(p[i]);
    } else if (t.dtype == "F16") {
        const uint16_t* p = reinterpret_cast<const uint16_t*>(t.data);
        for (int64_t i = 0; i < n; ++i) out[i] = f16_bits_to_float(p[i]);
    } else {
        throw WeightsError(dir_ + ": tensor '" + spec.name + "' must be floating point (F32, BF16 or F16), found " + t.dtype);
    }
}

RandomSource::RandomSource(uint64_t seed, const std::string& weights_dtype) : seed_(seed) {
    if (weights_dtype != "bfloat16" && weights_dtype != "float32")
        throw WeightsError("random weights are stored as bfloat16 or float32, not '" + weights_dtype + "'");
    round_bf16_ = weights_dtype == "bfloat16";
}

void RandomSource::read(const ParamSpec& spec, const std::string&, std::vector<float>& out) const {
    int64_t n = 1;
    for (int64_t s : spec.shape) n *= s;
    out.resize(static_cast<size_t>(n));
    normal_values(seed_, spec.name, 0, n, spec.mean, spec.std, out.data());
    if (round_bf16_ && spec.role == ParamSpec::Matrix)
        for (auto& v : out) v = bf16_bits_to_float(float_to_bf16_bits(v));
}

// ---------------------------------------------------------------------------------------------
// device tensors
// ---------------------------------------------------------------------------------------------
DeviceTensors::~DeviceTensors() {
    for (void* p : ptrs_) (void)hipFree(p);
}

void* DeviceTensors::allocate(size_t bytes, bool zero) {
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, std::max<size_t>(bytes, 16));
    if (e != hipSuccess) throw WeightsError("hipMalloc of " + std::to_string(bytes) + " bytes failed: " + hipGetErrorString(e));
    if (zero) {
        e = hipMemset(p, 0, std::max<size_t>(bytes, 16));
        if (e != hipSuccess) throw WeightsError(std::string("hipMemset failed: ") + hipGetErrorString(e));
    }
    ptrs_.push_back(p);
    bytes_ += bytes;
    return p;
}

Tensor2 DeviceTensors::upload(const std::vector<float>& values, int64_t rows, int64_t cols, int dtype) {
    const size_t n = static_cast<size_t>(rows) * cols;
    if (values.size() != n) throw WeightsError("upload: size mismatch");
    void* dev = allocate(n * dtype_size(dtype), false);
    hipError_t e;
    if (dtype == F32) {
        e = hipMemcpy(dev, values.data(), n * 4, hipMemcpyHostToDevice);
    } else {
        std::vector<uint16_t> half(n);
        for (size_t i = 0; i < n; ++i) half[i] = float_to_bf16_bits(values[i]);
        e = hipMemcpy(dev, half.data(), n * 2, hipMemcpyHostToDevice);
    }
    if (e != hipSuccess) throw WeightsError(std::string("copy to the device failed: ") + hipGetErrorString(e));
    return Tensor2(dev, dtype, rows, cols);
}

// ---------------------------------------------------------------------------------------------
// loading
// ---------------------------------------------------------------------------------------------
static std::string shape_text(const std::vector<int64_t>& s) {
    std::string t = "[";
    for (size_t i = 0; i < s.size(); ++i) t += (i ? ", " : "") + std::to_string(s[i]);
    return t + "]";
}

std::map<std::string, std::string> check_checkpoint(const std::vector<ParamSpec>& specs, const TensorSource& source,
                                                    const std::vector<std::string>& optional_prefixes,
                                                    const std::function<bool(const std::string&)>& ignored,
                                                    const std::string& where) {
    std::map<std::string, const ParamSpec*> by_name;
    for (const auto& s : specs) by_name[s.name] = &s;
    std::map<std::string, std::string> available;     // short name -> stored name
    {
        for (const std::string& name : source.names()) {
            std::string short_name = name;
            if (!by_name.count(name)) {
                for (const auto& p : optional_prefixes)
                    if (name.compare(0, p.size(), p) == 0) { short_name = name.substr(p.size()); break; }
            }
            if (ignored && ignored(short_name)) continue;
            available[short_name] = name;
        }
        std::vector<std::string> missing, unexpected, wrong;
        for (const auto& s : specs) {
            auto it = available.find(s.name);
            if (it == available.end()) { missing.push_back(s.name); continue; }
            const std::vector<int64_t>* shape = source.shape_of(it->second);
            if (shape == nullptr || *shape != s.shape)
                wrong.push_back(s.name + ": expected " + shape_text(s.shape) + ", found " + (shape ? shape_text(*shape) : "nothing"));
        }
        for (const auto& kv : available)
            if (!by_name.count(kv.first)) unexpected.push_back(kv.first);
        if (!missing.empty() || !unexpected.empty() || !wrong.empty()) {
            auto join = [](const std::vector<std::string>& v, const char* sep) {
                std::string t;
                for (size_t i = 0; i < v.size(); ++i) t += (i ? sep : "") + v[i];
                return t;
            };
            std::string msg = where + ": the checkpoint does not fit the model";
            if (!missing.empty()) msg += "\n  missing tensors (" + std::to_string(missing.size()) + "): " + join(missing, ", ");
            if (!unexpected.empty()) msg += "\n  unexpected tensors (" + std::to_string(unexpected.size()) + "): " + join(unexpected, ", ");
            if (!wrong.empty()) msg += "\n  wrong shapes (" + std::to_string(wrong.size()) + "): " + join(wrong, "; ");
            throw WeightsError(msg);
        }
    }
    return available;
}

std::map<std::string, Tensor2> load_tensors(const std::vector<ParamSpec>& specs, const TensorSource& source,
                                            int compute_dtype, DeviceTensors& store,
                                            const std::vector<std::string>& optional_prefixes,
                                            const std::function<bool(const std::string&)>& ignored,
                                            const std::string& where) {
    std::map<std::string, std::string> available;     // short name -> stored name
    if (!source.generates()) available = check_checkpoint(specs, source, optional_prefixes, ignored, where);
    std::map<std::string, Tensor2> out;
    std::vector<float> values, turned;
    for (const auto& s : specs) {
        source.read(s, source.generates() ? s.name : available.at(s.name), values);
        int64_t rows = 1, cols = 1;
        if (s.shape.size() == 1) cols = s.shape[0];
        else if (s.shape.size() == 2) { rows = s.shape[0]; cols = s.shape[1]; }
        else throw WeightsError(where + ": tensor '" + s.name + "' has " + std::to_string(s.shape.size()) + " dimensions; one or two are expected");
        const std::vector<float>* src = &values;
        if (s.transpose) {
            turned.resize(values.size());
            for (int64_t r = 0; r < rows; ++r)
                for (int64_t c = 0; c < cols; ++c) turned[static_cast<size_t>(c) * rows + r] = values[static_cast<size_t>(r) * cols + c];
            std::swap(rows, cols);
            src = &turned;
        }
        out[s.name] = store.upload(*src, rows, cols, s.role == ParamSpec::Matrix ? compute_dtype : F32);
    }
    return out;
}

void write_random_model(const std::string& out_dir, const Json& config, const std::vector<ParamSpec>& specs,
                        uint64_t seed, const std::string& weights_dtype) {
    RandomSource src(seed, weights_dtype);
    std::map<std::string, TensorToStore> tensors;
    std::vector<float> values;
    for (const auto& s : specs) {
        src.read(s, s.name, values);
        TensorToStore t;
        t.shape = s.shape;
        if (s.role == ParamSpec::Matrix && weights_dtype == "bfloat16") {
            t.dtype = "BF16";
            t.bytes.resize(values.size() * 2);
            uint16_t* p = reinterpret_cast<uint16_t*>(t.bytes.data());
            for (size_t i = 0; i < values.size(); ++i) p[i] = float_to_bf16_bits(values[i]);
        } else {
            t.dtype = "F32";
            t.bytes.resize(values.size() * 4);
            std::memcpy(t.bytes.data(), values.data(), values.size() * 4);
        }
        tensors.emplace(s.name, std::move(t));
    }
    ::mkdir(out_dir.c_str(), 0755);
    Json cfg = config;
    cfg.set("torch_dtype", Json::of(weights_dtype));
    std::ofstream f(out_dir + "/config.json");
    if (!f) throw WeightsError(out_dir + "/config.json: cannot be written");
    f << cfg.dump() << "\n";
    save_safetensors(out_dir + "/model.safetensors", tensors, {{"format", "pt"}, {"seed", std::to_string(seed)}});
}

}  // namespace minillm
