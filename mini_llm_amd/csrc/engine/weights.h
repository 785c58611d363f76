// Weights for the native engine: a safetensors reader and writer, the specified random generator,
// and the loader that fills a model's tensors by name and reports every mismatch in one error.
//
// The reference reads one raw fp32 file per tensor with no shape information
// (/root/reference/src/model/gpt2_model.cu:32-70,115-173); a model folder here holds config.json and
// model.safetensors (or shards named by model.safetensors.index.json).
#pragma once

#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "json.h"
#include "ops.h"

namespace minillm {

class WeightsError : public std::runtime_error {
public:
    explicit WeightsError(const std::string& what) : std::runtime_error(what) {}
};

// ---- safetensors ---------------------------------------------------------------------------------
struct StoredTensor {
    std::string dtype;               // "F32", "BF16", "F16"
    std::vector<int64_t> shape;
    const unsigned char* data = nullptr;
    size_t bytes = 0;
    // the product of the dimensions; -1 if one is negative or the product does not fit 63 bits
    int64_t numel() const {
        int64_t n = 1;
        for (int64_t s : shape) {
            if (s < 0 || (s != 0 && n > INT64_MAX / s)) return -1;
            n *= s;
        }
        return n;
    }
};

// 8-byte little-endian header length, a JSON header {name: {dtype, shape, data_offsets}}
// ("__metadata__" is skipped), then the raw little-endian data; the file is memory-mapped.
class SafetensorsFile {
public:
    explicit SafetensorsFile(const std::string& path);
    ~SafetensorsFile();
    SafetensorsFile(const SafetensorsFile&) = delete;
    SafetensorsFile& operator=(const SafetensorsFile&) = delete;
    const std::map<std::string, StoredTensor>& tensors() const { return tensors_; }
    const std::string& path() const { return path_; }

private:
    std::string path_;
    void* map_ = nullptr;
    size_t size_ = 0;
    std::map<std::string, StoredTensor> tensors_;
};

// Writes name -> (dtype, shape, bytes), names in sorted order.
struct TensorToStore {
    std::string dtype;
    std::vector<int64_t> shape;
    std::vector<unsigned char> bytes;
};
void save_safetensors(const std::string& path, const std::map<std::string, TensorToStore>& tensors,
                      const std::map<std::string, std::string>& metadata);

// ---- the random-weights generator ----------------------------------------------------------------
// Element i of the tensor called `name` under `seed`:
//   key = splitmix64(seed) ^ fnv1a64(name);  a = splitmix64(key + 2i),  b = splitmix64(key + 2i + 1)
//   u1 = ((a >> 11) + 1) / 2^53,  u2 = (b >> 11) / 2^53,  z = sqrt(-2 ln u1) cos(2 pi u2)  (float64)
//   value = float32(mean + std z)
// A value depends on (seed, name, index) only; any program that follows this draws the same values.
uint64_t splitmix64(uint64_t x);
uint64_t fnv1a64(const std::string& s);
void normal_values(uint64_t seed, const std::string& name, int64_t first, int64_t n, double mean, double std,
                   float* out);

// bfloat16 <-> float32, round to nearest even
uint16_t float_to_bf16_bits(float f);
float bf16_bits_to_float(uint16_t b);
float f16_bits_to_float(uint16_t h);

// ---- what a model asks of its checkpoint -----------------------------------------------------------
// One tensor a model expects: its name and shape as stored, how it is kept (role), how it is laid out,
// and the distribution of the random-weights mode.
struct ParamSpec {
    std::string name;
    std::vector<int64_t> shape;          // as stored in the checkpoint
    enum Role { Matrix, Vector } role;   // matrix: kept in the compute dtype; vector: kept in fp32
    bool transpose = false;              // stored [in, out], used as [out, in]
    double mean = 0.0, std = 0.02;
};

// Where tensors come from: a checkpoint on disk or the random generator. Gives fp32 host values.
class TensorSource {
public:
    virtual ~TensorSource() = default;
    // names the source holds (a random source holds every name it is asked for: empty list)
    virtual std::vector<std::string> names() const = 0;
    virtual bool generates() const { return false; }
    // shape of a stored tensor, or nullptr if the source does not hold it
    virtual const std::vector<int64_t>* shape_of(const std::string& name) const = 0;
    // the tensor as float32 values, row-major as stored
    virtual void read(const ParamSpec& spec, const std::string& stored_name, std::vector<float>& out) const = 0;
};

class CheckpointSource final : public TensorSource {
public:
    explicit CheckpointSource(const std::string& model_dir);     // model.safetensors, or the shards of the index
    std::vector<std::string> names() const override;
    const std::vector<int64_t>* shape_of(const std::string& name) const override;
    void read(const ParamSpec& spec, const std::string& stored_name, std::vector<float>& out) const override;

private:
    std::string dir_;
    std::vector<std::unique_ptr<SafetensorsFile>> files_;
    std::map<std::string, const StoredTensor*> all_;
};

// Random weights: matrices rounded to `weights_dtype` ("bfloat16": what a written folder would store,
// so that the 32-bit and the bfloat16 path read identical values; or "float32").
class RandomSource final : public TensorSource {
public:
    RandomSource(uint64_t seed, const std::string& weights_dtype);
    std::vector<std::string> names() const override { return {}; }
    bool generates() const override { return true; }
    const std::vector<int64_t>* shape_of(const std::string&) const override { return nullptr; }
    void read(const ParamSpec& spec, const std::string& stored_name, std::vector<float>& out) const override;

private:
    uint64_t seed_;
    bool round_bf16_;
};

// Device memory that a loaded model owns.
class DeviceTensors {
public:
    DeviceTensors() = default;
    ~DeviceTensors();
    DeviceTensors(const DeviceTensors&) = delete;
    DeviceTensors& operator=(const DeviceTensors&) = delete;
    // Uploads float32 host values [rows, cols] as `dtype` (bf16: round to nearest even) and returns the view.
    Tensor2 upload(const std::vector<float>& values, int64_t rows, int64_t cols, int dtype);
    void* allocate(size_t bytes, bool zero);
    size_t bytes() const { return bytes_; }

private:
    std::vector<void*> ptrs_;
    size_t bytes_ = 0;
};

// Compares what a checkpoint holds with what the model expects (names, with an optional prefix accepted and
// `ignored` names skipped; shapes) and returns spec name -> stored name. ONE WeightsError lists missing,
// unexpected and wrong-shape tensors. Touches no device.
std::map<std::string, std::string> check_checkpoint(const std::vector<ParamSpec>& specs, const TensorSource& source,
                                                    const std::vector<std::string>& optional_prefixes,
                                                    const std::function<bool(const std::string&)>& ignored,
                                                    const std::string& where);

// Looks every spec up in the source (an optional name prefix is accepted, `ignored` names are skipped),
// checks shapes, converts (matrices -> compute dtype, transposed once if stored [in, out]; vectors -> fp32)
// and uploads. ONE WeightsError lists missing, unexpected and wrong-shape tensors.
std::map<std::string, Tensor2> load_tensors(const std::vector<ParamSpec>& specs, const TensorSource& source,
                                            int compute_dtype, DeviceTensors& store,
                                            const std::vector<std::string>& optional_prefixes,
                                            const std::function<bool(const std::string&)>& ignored,
                                            const std::string& where);

// Writes config.json and model.safetensors for the specs from the random generator.
void write_random_model(const std::string& out_dir, const Json& config, const std::vector<ParamSpec>& specs,
                        uint64_t seed, const std::string& weights_dtype);

}  // namespace minillm
