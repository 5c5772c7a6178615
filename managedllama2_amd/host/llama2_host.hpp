// C++ host layer over the C ABI (include/llama2_hip.h): the classes of the
// reference's C# library libLlama2 for the decode path, name for name --
// Config, QWeight, PerLayerWeight, TransformerWeights, RunState, Module and the
// eleven module classes, Sampler (greedy branch), Transformer (ITransformer on
// token ids).  Device memory and launches come from libllama2_hip.so where the
// reference gets them from ManagedCuda.  Header-only; errors are exceptions
// (the reference's CudaException / FileLoadException / NotImplementedException).
#pragma once

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include "../../include/llama2_hip.h"

namespace libLlama2 {

using Half = llama2_half;

struct Llama2Exception : std::runtime_error { // CudaException
    int code;
    Llama2Exception(int c, const std::string& m) : std::runtime_error(m), code(c) {}
};
struct FileLoadException : std::runtime_error {
    using std::runtime_error::runtime_error;
};
struct NotImplementedException : std::logic_error {
    using std::logic_error::logic_error;
};

inline void Check(int status)
{
    if (status != LLAMA2_OK)
        throw Llama2Exception(status, llama2_last_error());
}

inline int CeilDiv(int a, int b) { return (a + (b - 1)) / b; } // src/Module.cs:24-25

// ---------------------------------------------------------------- src/Config.cs:6-39
struct Config : llama2_config {
    static constexpr size_t Size = 32;

    static Config LoadConfig(const void* bytes, size_t available)
    {
        if (available < Size)
            throw FileLoadException("Invalid model config");
        Config c;
        std::memcpy(static_cast<llama2_config*>(&c), bytes, Size);
        if (c.rope_theta != 10000.0f) // :27-28
            throw FileLoadException("Invalid model config");
        c.Validate();
        return c;
    }
    // The header comes from a file: nothing is derived from it (kvDim divides by n_heads, the sizes
    // of the tensor stream multiply its fields) before every field is known to be sane.  The
    // reference trusts the header and fails later with an arithmetic or a file-length exception;
    // here a bad field is the same "Invalid model config" as a bad rope_theta.
    void Validate() const
    {
        constexpr int kMaxWidth = 1 << 20, kMaxLayers = 1 << 12, kMaxVocab = 1 << 24, kMaxSeq = 1 << 24;
        const bool ok = dim > 0 && dim <= kMaxWidth && hidden_dim > 0 && hidden_dim <= kMaxWidth && n_layers > 0 &&
                        n_layers <= kMaxLayers && n_heads > 0 && n_heads <= dim && dim % n_heads == 0 && n_kv_heads > 0 &&
                        n_kv_heads <= n_heads && n_heads % n_kv_heads == 0 && vocab_size > 0 && vocab_size <= kMaxVocab &&
                        seq_len > 0 && seq_len <= kMaxSeq;
        if (!ok)
            throw FileLoadException("Invalid model config");
    }
    int kvDim() const { return static_cast<int>(static_cast<long long>(dim) * n_kv_heads / n_heads); }
};
static_assert(sizeof(llama2_config) == 32, "the model-file header is 32 bytes");

// ---------------------------------------------------------------- CudaDeviceVariable<T>
template <class T>
class DeviceVariable {
  public:
    DeviceVariable() = default;
    explicit DeviceVariable(size_t size) : size_(size) { Check(llama2_malloc(&ptr_, size * sizeof(T))); }
    DeviceVariable(const T* host, size_t size) : DeviceVariable(size) { CopyToDevice(host, size, 0); } // implicit T[] ->
    // A window of `size` elements into memory another DeviceVariable owns (never freed from here).
    static DeviceVariable Window(void* ptr, size_t size)
    {
        DeviceVariable v;
        v.ptr_ = ptr;
        v.size_ = size;
        v.owns_ = false;
        return v;
    }
    DeviceVariable(const DeviceVariable&) = delete;
    DeviceVariable& operator=(const DeviceVariable&) = delete;
    DeviceVariable(DeviceVariable&& o) noexcept : ptr_(o.ptr_), size_(o.size_), owns_(o.owns_) { o.ptr_ = nullptr; }
    DeviceVariable& operator=(DeviceVariable&& o) noexcept
    {
        std::swap(ptr_, o.ptr_);
        std::swap(size_, o.size_);
        std::swap(owns_, o.owns_);
        return *this;
    }
    ~DeviceVariable()
    {
        if (ptr_ && owns_)
            llama2_free(ptr_);
    }
    T* DevicePointer() const { return static_cast<T*>(ptr_); }
    size_t Size() const { return size_; }
    static constexpr size_t TypeSize = sizeof(T);
    T* OffsetPointer(size_t offset) const { return DevicePointer() + offset; } // src/Extensions.cs:20-21
    void CopyToDevice(const T* source, size_t count, size_t position = 0)     // src/Extensions.cs:23-24
    {
        Check(llama2_memcpy_h2d(ptr_, position * sizeof(T), source, count * sizeof(T)));
    }
    std::vector<T> ToHost() const // explicit CudaDeviceVariable<T> -> T[]
    {
        std::vector<T> out(size_);
        Check(llama2_memcpy_d2h(out.data(), ptr_, 0, size_ * sizeof(T)));
        return out;
    }
    T operator[](size_t index) const // the synchronising 1-element read of src/Sampler.cs:69
    {
        T v;
        Check(llama2_memcpy_d2h(&v, ptr_, index * sizeof(T), sizeof(T)));
        return v;
    }
    void Zero() { Check(llama2_memset(ptr_, 0, size_ * sizeof(T))); }

  private:
    void* ptr_ = nullptr;
    size_t size_ = 0;
    bool owns_ = true;
};

// ---------------------------------------------------------------- src/QWeight.cs:5-10
struct QWeight {
    DeviceVariable<uint32_t> Weight;
    DeviceVariable<uint32_t> Zeros;
    DeviceVariable<Half> Scales;
    llama2_qweight View() const { return {Weight.DevicePointer(), Zeros.DevicePointer(), Scales.DevicePointer()}; }
};

// ---------------------------------------------------------------- src/PerLayerWeight.cs:5-16
struct PerLayerWeight {
    DeviceVariable<Half> rmsAttentionWeight, rmsFeedForwardWeight;
    QWeight queryWeight, keyWeight, valueWeight, outputWeight, gateWeight, upWeight, downWeight;
};

// A read-only mapping of the model file (MemoryMappedFile in the reference).
class MappedFile {
  public:
    explicit MappedFile(const std::string& path)
    {
        fd_ = ::open(path.c_str(), O_RDONLY);
        if (fd_ < 0)
            throw FileLoadException("cannot open " + path);
        struct stat st;
        if (fstat(fd_, &st) != 0 || st.st_size <= 0) {
            ::close(fd_);
            throw FileLoadException("cannot stat " + path);
        }
        size_ = static_cast<size_t>(st.st_size);
        data_ = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
        if (data_ == MAP_FAILED) {
            ::close(fd_);
            throw FileLoadException("cannot map " + path);
        }
    }
    MappedFile(const MappedFile&) = delete;
    ~MappedFile()
    {
        munmap(data_, size_);
        ::close(fd_);
    }
    const uint8_t* data() const { return static_cast<const uint8_t*>(data_); }
    size_t size() const { return size_; }

  private:
    int fd_ = -1;
    void* data_ = nullptr;
    size_t size_ = 0;
};

// ---------------------------------------------------------------- src/TransformerWeights.cs:6-104
class TransformerWeights {
  public:
    DeviceVariable<Half> tokenEmbeddingTable, classifierWeights, rmsFinalWeight;
    std::vector<PerLayerWeight> layers;

    // Bytes the tensor stream must have for this config (the `offset != remaining` check, :39-40).
    static size_t ExpectedBytes(const Config& c)
    {
        const size_t dim = c.dim, hidden = c.hidden_dim, kv = c.kvDim();
        auto q = [](size_t rows, size_t cols) {
            const size_t ss = (rows + 127) / 128, ws = (rows + 31) / 32 * 4, zs = (ss + 7) / 8;
            return cols * (ws * 4 + zs * 4 + ss * 2);
        };
        const size_t layer = q(dim, dim) + 2 * q(dim, kv) + q(dim, dim) + 2 * q(dim, hidden) + q(hidden, dim) + 4 * dim;
        return 2 * (2 * static_cast<size_t>(c.vocab_size) * dim + dim) + c.n_layers * layer;
    }

    TransformerWeights(const Config& config, const MappedFile& file) : config_(config)
    {
        const size_t remaining = file.size() - Config::Size;
        if (ExpectedBytes(config) != remaining)
            throw FileLoadException("Failed to read file. offset: " + std::to_string(ExpectedBytes(config)) +
                                    " != length: " + std::to_string(remaining));
        // One allocation for the whole tensor stream (the reference allocates per tensor): the mat-vec
        // kernels stream 3 % faster when a layer's tensors are neighbours in the address space.
        const size_t tensors = 3 + static_cast<size_t>(config.n_layers) * (7 * 3 + 2);
        arena_ = DeviceVariable<uint8_t>(remaining + tensors * kAlign);
        const uint8_t* p = file.data() + Config::Size;
        const size_t vd = static_cast<size_t>(config.vocab_size) * config.dim;
        tokenEmbeddingTable = ReadWeight(p, vd);
        classifierWeights = ReadWeight(p, vd);
        rmsFinalWeight = ReadWeight(p, config.dim);
        layers.reserve(config.n_layers);
        const int dim = config.dim, hidden = config.hidden_dim, kv = config.kvDim();
        for (int i = 0; i < config.n_layers; ++i) { // ReadLayer, :84-94: q, k, v, o, up, gate, down, norms
            PerLayerWeight L;
            L.queryWeight = ReadQWeight(p, dim, dim);
            L.keyWeight = ReadQWeight(p, dim, kv);
            L.valueWeight = ReadQWeight(p, dim, kv);
            L.outputWeight = ReadQWeight(p, dim, dim);
            L.upWeight = ReadQWeight(p, dim, hidden);
            L.gateWeight = ReadQWeight(p, dim, hidden);
            L.downWeight = ReadQWeight(p, hidden, dim);
            L.rmsAttentionWeight = ReadWeight(p, dim);
            L.rmsFeedForwardWeight = ReadWeight(p, dim);
            layers.push_back(std::move(L));
        }
    }

    std::vector<llama2_layer_weights> LayerViews() const
    {
        std::vector<llama2_layer_weights> v;
        for (const PerLayerWeight& L : layers)
            v.push_back({L.queryWeight.View(), L.keyWeight.View(), L.valueWeight.View(), L.outputWeight.View(),
                         L.gateWeight.View(), L.upWeight.View(), L.downWeight.View(),
                         L.rmsAttentionWeight.DevicePointer(), L.rmsFeedForwardWeight.DevicePointer()});
        return v;
    }

  private:
    static constexpr size_t kAlign = 256;
    template <class T>
    DeviceVariable<T> Read(const uint8_t*& p, size_t size)
    {
        DeviceVariable<T> v = DeviceVariable<T>::Window(arena_.DevicePointer() + used_, size);
        v.CopyToDevice(reinterpret_cast<const T*>(p), size, 0);
        used_ += (size * sizeof(T) + kAlign - 1) / kAlign * kAlign;
        p += size * sizeof(T);
        return v;
    }
    DeviceVariable<Half> ReadWeight(const uint8_t*& p, size_t size) { return Read<Half>(p, size); }
    DeviceVariable<uint32_t> ReadIntArray(const uint8_t*& p, size_t size) { return Read<uint32_t>(p, size); }
    QWeight ReadQWeight(const uint8_t*& p, int rows, int cols) // :54-69
    {
        const int scalesSize = CeilDiv(rows, 128), weightsSize = CeilDiv(rows, 32) * 4, zerosSize = CeilDiv(scalesSize, 8);
        QWeight q;
        q.Weight = ReadIntArray(p, static_cast<size_t>(weightsSize) * cols);
        q.Zeros = ReadIntArray(p, static_cast<size_t>(zerosSize) * cols);
        q.Scales = ReadWeight(p, static_cast<size_t>(scalesSize) * cols);
        return q;
    }
    Config config_;
    DeviceVariable<uint8_t> arena_;
    size_t used_ = 0;
};

// ---------------------------------------------------------------- src/RunState.cs:5-55
struct RunState {
    DeviceVariable<Half> x, xb, h, q, attention, logits, keyCache, valueCache;
    DeviceVariable<int> tokens, indices;

    RunState(Config& config, int kvDim)
    {
        auto maxUsableSequence = [&]() { // CalculateMaxUsableSequence, :29-39
            const size_t kernelMem = 8u * 1024 * 1024;
            size_t free_bytes = 0, total = 0;
            Check(llama2_mem_info(&free_bytes, &total));
            const size_t remaining = free_bytes > kernelMem ? free_bytes - kernelMem : 0;
            const size_t required = static_cast<size_t>(config.n_layers) * kvDim * sizeof(Half) * 2 + sizeof(int) +
                                    static_cast<size_t>(config.vocab_size) * sizeof(int);
            const size_t fit = remaining / required;
            return static_cast<int>(fit < static_cast<size_t>(config.seq_len) ? fit : config.seq_len);
        };
        x = DeviceVariable<Half>(config.dim);
        xb = DeviceVariable<Half>(config.dim);
        h = DeviceVariable<Half>(config.hidden_dim);
        q = DeviceVariable<Half>(config.dim);
        const int span = config.dim > config.seq_len ? config.dim : config.seq_len;
        attention = DeviceVariable<Half>(static_cast<size_t>(config.n_heads) * span);
        logits = DeviceVariable<Half>(config.vocab_size);
        config.seq_len = maxUsableSequence(); // :48
        const size_t kv = static_cast<size_t>(config.n_layers) * config.seq_len * kvDim;
        keyCache = DeviceVariable<Half>(kv);
        valueCache = DeviceVariable<Half>(kv);
        tokens = DeviceVariable<int>(config.seq_len + 1);
        indices = DeviceVariable<int>(config.vocab_size); // :53
        keyCache.Zero();
        valueCache.Zero();
        tokens.Zero();
    }
    llama2_run_state View() const
    {
        return {x.DevicePointer(), xb.DevicePointer(), h.DevicePointer(), q.DevicePointer(), attention.DevicePointer(),
                logits.DevicePointer(), keyCache.DevicePointer(), valueCache.DevicePointer(), tokens.DevicePointer(),
                indices.DevicePointer()};
    }
};

// ---------------------------------------------------------------- src/Module.cs and the module classes
class Module {
  public:
    explicit Module(const Config* config = nullptr) : config_(config) {}

  protected:
    const Config* config_;
    static void Sizes(int rows, int& zerosSize, int& scalesSize, int& weightsSize)
    {
        scalesSize = CeilDiv(rows, 128);
        weightsSize = CeilDiv(rows, 32) * 4;
        zerosSize = CeilDiv(scalesSize, 8);
    }
};

struct MatVec : Module { // src/MatVec.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& output, DeviceVariable<Half>& input, DeviceVariable<Half>& matrix, int rows, int cols)
    {
        Check(llama2_mat_vec(output.DevicePointer(), input.DevicePointer(), matrix.DevicePointer(), rows, cols));
    }
};

struct QKVMatVec : Module { // src/QKVMatVec.cs
    int kvDim = 0;
    QKVMatVec() = default;
    explicit QKVMatVec(const Config* c) : Module(c), kvDim(c->kvDim()) {}
    void Forward(DeviceVariable<Half>& queryOutput, DeviceVariable<Half>& keyOutput, DeviceVariable<Half>& valueOutput,
                 DeviceVariable<Half>& input, QWeight& query, QWeight& key, QWeight& value, int rows, int cols,
                 size_t layerOffset, int pos)
    {
        int zs, ss, ws;
        Sizes(rows, zs, ss, ws);
        const size_t offset = layerOffset + static_cast<size_t>(pos) * kvDim;
        Check(llama2_qkv_mat_vec(queryOutput.DevicePointer(), keyOutput.OffsetPointer(offset), valueOutput.OffsetPointer(offset),
                                 input.DevicePointer(), query.Weight.DevicePointer(), query.Zeros.DevicePointer(),
                                 query.Scales.DevicePointer(), key.Weight.DevicePointer(), key.Zeros.DevicePointer(),
                                 key.Scales.DevicePointer(), value.Weight.DevicePointer(), value.Zeros.DevicePointer(),
                                 value.Scales.DevicePointer(), rows, cols, zs, ss, ws));
    }
};

struct MatVecSwiGLU : Module { // src/MatVecSwiGLU.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& output, DeviceVariable<Half>& input, QWeight& g, QWeight& u, int rows, int cols)
    {
        int zs, ss, ws;
        Sizes(rows, zs, ss, ws);
        Check(llama2_mat_vec_swiglu(output.DevicePointer(), input.DevicePointer(), g.Weight.DevicePointer(),
                                    g.Zeros.DevicePointer(), g.Scales.DevicePointer(), u.Weight.DevicePointer(),
                                    u.Zeros.DevicePointer(), u.Scales.DevicePointer(), rows, cols, zs, ss, ws));
    }
};

struct MatVecResidual : Module { // src/MatVecResidual.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& output, DeviceVariable<Half>& input, QWeight& matrix, int rows, int cols)
    {
        int zs, ss, ws;
        Sizes(rows, zs, ss, ws);
        Check(llama2_mat_vec_residual_int4(output.DevicePointer(), input.DevicePointer(), matrix.Weight.DevicePointer(),
                                           matrix.Zeros.DevicePointer(), matrix.Scales.DevicePointer(), rows, cols, zs, ss, ws));
    }
};

struct MatVecStrided : Module { // src/MatVecStrided.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& attention, DeviceVariable<Half>& query, DeviceVariable<Half>& key, int headSize,
                 int dim, int seqLength, size_t layerOffset, float scale)
    {
        Check(llama2_mat_vec_strided(attention.DevicePointer(), query.DevicePointer(), key.OffsetPointer(layerOffset), headSize,
                                     seqLength, headSize, headSize, dim, seqLength, scale, config_->n_heads));
    }
};

struct VecMat : Module { // src/VecMat.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& output, DeviceVariable<Half>& value, DeviceVariable<Half>& attention, int headSize,
                 int dim, int seqLength, size_t layerOffset)
    {
        Check(llama2_vec_mat(output.DevicePointer(), attention.DevicePointer(), value.OffsetPointer(layerOffset), headSize,
                             seqLength, headSize, headSize, dim, config_->n_heads));
    }
};

struct RMSNorm : Module { // src/RMSNorm.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& output, DeviceVariable<Half>& input, DeviceVariable<Half>& weights, int size,
                 float eps = 1e-5f)
    {
        Check(llama2_rmsnorm(output.DevicePointer(), input.DevicePointer(), weights.DevicePointer(), size, eps));
    }
};

struct RoPERotation : Module { // src/RoPERotation.cs
    int kvDim = 0;
    RoPERotation() = default;
    explicit RoPERotation(const Config* c) : Module(c), kvDim(c->kvDim()) {}
    void Forward(DeviceVariable<Half>& query, DeviceVariable<Half>& key, int numKVHeads, int headSize, int pos,
                 size_t layerOffset, float theta)
    {
        const size_t offset = layerOffset + static_cast<size_t>(pos) * kvDim;
        Check(llama2_rope(query.DevicePointer(), key.OffsetPointer(offset), numKVHeads, headSize, pos, theta, config_->n_heads));
    }
};

struct Softmax : Module { // src/Softmax.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& attention, int seqLength)
    {
        Check(llama2_softmax(attention.DevicePointer(), seqLength, config_->n_heads));
    }
};

struct Argmax : Module { // src/Argmax.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& logits, int vocabSize, DeviceVariable<int>& tokens, int nextPos, bool generateToken)
    {
        Check(llama2_argmax(logits.DevicePointer(), vocabSize, tokens.DevicePointer(), nextPos, generateToken ? 1 : 0));
    }
};

struct Embedding : Module { // src/Embedding.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& output, DeviceVariable<Half>& table, int size, DeviceVariable<int>& tokens, int pos)
    {
        Check(llama2_embedding(output.DevicePointer(), table.DevicePointer(), size, tokens.DevicePointer(), pos));
    }
};

struct SoftmaxLogits : Module { // src/SoftmaxLogits.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& logits, int size, float temperature, DeviceVariable<int>& indices)
    {
        Check(llama2_softmax_logits(logits.DevicePointer(), size, temperature, indices.DevicePointer()));
    }
};

struct Sort : Module { // src/Sort.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& logits, DeviceVariable<int>& indices, int size)
    {
        Check(llama2_sort(logits.DevicePointer(), indices.DevicePointer(), size));
    }
};

struct CumulativeSum : Module { // src/CumulativeSum.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& logits, int size) { Check(llama2_cumulative_sum(logits.DevicePointer(), size)); }
};

struct SampleTopP : Module { // src/SampleTopP.cs
    using Module::Module;
    void Forward(DeviceVariable<Half>& logits, DeviceVariable<int>& indices, int size, float threshold,
                 DeviceVariable<int>& tokens, int nextPos)
    {
        Check(llama2_sample_top_p(logits.DevicePointer(), indices.DevicePointer(), size, threshold, tokens.DevicePointer(),
                                  nextPos));
    }
};

// ---------------------------------------------------------------- src/Sampler.cs
class Sampler {
  public:
    Sampler(const Config& config, RunState& runstate, float temperature, float topP, uint64_t seed)
        : config_(config), runstate_(runstate), temperature_(temperature), topP_(topP), seed_(seed), argmax_(&config_),
          softmax_(&config_), cumulativeSum_(&config_), sampleTopP_(&config_), sort_(&config_)
    {
    }
    float Temperature() const { return temperature_; }
    float TopP() const { return topP_; }
    // The reference draws from an unseeded System.Random (:24, :42); here the coin of a position is the
    // library's seeded stream, so a run can be reproduced (and matches llama2_decode_run_sampled).
    float Coin(int nextPosition) const { return llama2_sampler_coin(seed_, nextPosition); }
    int Sample(int nextPosition, bool generateToken)
    {
        const float coin = Coin(nextPosition); // :42
        RunState& rs = runstate_;
        const int n = config_.vocab_size;
        if (temperature_ == 0.0f || !generateToken) {
            argmax_.Forward(rs.logits, n, rs.tokens, nextPosition, generateToken); // :44-47
        } else {
            softmax_.Forward(rs.logits, n, temperature_, rs.indices); // :50
            float threshold;
            if (topP_ <= 0 || topP_ >= 1) {
                threshold = coin; // :53-55
            } else {
                sort_.Forward(rs.logits, rs.indices, n); // :59
                threshold = coin * topP_;                // :61
            }
            cumulativeSum_.Forward(rs.logits, n);                                              // :64
            sampleTopP_.Forward(rs.logits, rs.indices, n, threshold, rs.tokens, nextPosition); // :66
        }
        return rs.tokens[nextPosition]; // :69
    }

  private:
    Config config_;
    RunState& runstate_;
    float temperature_, topP_;
    uint64_t seed_;
    Argmax argmax_;
    SoftmaxLogits softmax_;
    CumulativeSum cumulativeSum_;
    SampleTopP sampleTopP_;
    Sort sort_;
};

// ---------------------------------------------------------------- src/ModelConverter.cs:196-328 (tensor side)
// RepackQWeightByName on host arrays: upload, repack on the GPU, download.  Reading the PyTorch
// checkpoint (zip + pickle) is outside this path; the caller brings the three tensors.
struct ModelConverter {
    enum class Format { v0, v1 };
    struct Repacked {
        std::vector<uint32_t> Weight, Zeros;
        std::vector<Half> Scales;
    };
    static int CeilDiv(int a, int b) { return (a + (b - 1)) / b; }
    static Repacked RepackQWeight(const uint32_t* qweight, const uint32_t* qzeros, const Half* scales, int height,
                                  int width, Format format)
    {
        const int groupSize = 128;
        const int scalesSize = CeilDiv(height, groupSize), weightsSize = CeilDiv(height, 8),
                  zerosSize = CeilDiv(scalesSize, 8);
        Repacked r;
        if (format == Format::v0) {
            const size_t w8 = static_cast<size_t>(CeilDiv(width, 8));
            DeviceVariable<uint32_t> wIn(qweight, w8 * height), wOut(static_cast<size_t>(weightsSize) * width);
            Check(llama2_repack_qdata(wOut.DevicePointer(), wIn.DevicePointer(), height, width)); // :238
            DeviceVariable<uint32_t> zIn(qzeros, w8 * scalesSize), zOut(static_cast<size_t>(zerosSize) * width);
            Check(llama2_repack_qdata(zOut.DevicePointer(), zIn.DevicePointer(), scalesSize, width)); // :239
            DeviceVariable<Half> sIn(scales, static_cast<size_t>(scalesSize) * width),
                sOut(static_cast<size_t>(scalesSize) * width);
            Check(llama2_repack_scales(sOut.DevicePointer(), sIn.DevicePointer(), scalesSize, width)); // :240
            r.Weight = wOut.ToHost();
            r.Zeros = zOut.ToHost();
            r.Scales = sOut.ToHost();
        } else {
            r.Weight.assign(qweight, qweight + static_cast<size_t>(weightsSize) * width);
            r.Zeros.assign(qzeros, qzeros + static_cast<size_t>(zerosSize) * width);
            DeviceVariable<Half> sIn(scales, static_cast<size_t>(zerosSize) * 8 * width),
                sOut(static_cast<size_t>(scalesSize) * width);
            Check(llama2_compact_scales_v1(sOut.DevicePointer(), sIn.DevicePointer(), scalesSize, width)); // :247-262
            r.Scales = sOut.ToHost();
        }
        return r;
    }
};

// ---------------------------------------------------------------- src/ITransformer.cs, src/Transformer.cs
struct ITransformer {
    virtual ~ITransformer() = default;
    // Generate on token ids (the tokenizer is outside this path): yields at most `steps` tokens.
    virtual std::vector<int> Generate(const std::vector<int>& promptTokens, int steps) = 0;
};

class Transformer : public ITransformer {
  public:
    enum Mode { HostLoop = -1, Modules = LLAMA2_DECODE_MODULES, Fused = LLAMA2_DECODE_FUSED,
                FusedGraph = LLAMA2_DECODE_FUSED | LLAMA2_DECODE_GRAPH };

    // temperature 0 is greedy decoding; the reference's defaults are temperature 0.5, topP 0.9 (:42)
    explicit Transformer(const std::string& modelPath, Mode mode = HostLoop, bool stopOnSpecial = true,
                         float temperature = 0.0f, float topP = 0.9f, uint64_t seed = 0)
        : stopOnSpecial_(stopOnSpecial)
    {
        Check(llama2_init(0)); // new CudaContext(deviceID), :48-49
        MappedFile file(modelPath);
        config = Config::LoadConfig(file.data(), file.size()); // :51
        kvDim = config.kvDim();
        if (kvDim != config.dim) // :55-56
            throw NotImplementedException("Differing kvDim dimention not currently supported.");
        weights = std::make_unique<TransformerWeights>(config, file);
        runstate = std::make_unique<RunState>(config, kvDim);
        sampler = std::make_unique<Sampler>(config, *runstate, temperature, topP, seed);
        embedding = Embedding(&config);
        rmsNorm = RMSNorm(&config);
        qkvMatVec = QKVMatVec(&config);
        rope = RoPERotation(&config);
        matVecStrided = MatVecStrided(&config);
        softmax = Softmax(&config);
        vecMat = VecMat(&config);
        matVecResidual = MatVecResidual(&config);
        matVecSwiGLU = MatVecSwiGLU(&config);
        matVec = MatVec(&config);
        if (mode != HostLoop) {
            layerViews_ = weights->LayerViews();
            llama2_transformer_weights w{weights->tokenEmbeddingTable.DevicePointer(), weights->classifierWeights.DevicePointer(),
                                         weights->rmsFinalWeight.DevicePointer(), layerViews_.data()};
            llama2_run_state s = runstate->View();
            Check(llama2_decode_create(&decoder_, &config, &w, &s, mode));
        }
    }
    ~Transformer() override
    {
        if (decoder_)
            llama2_decode_destroy(decoder_);
    }

    std::vector<int> Generate(const std::vector<int>& promptTokens, int steps) override // :89-112
    {
        std::vector<int> out;
        runstate->tokens.CopyToDevice(promptTokens.data(), promptTokens.size());
        for (int pos = 0; pos < steps; ++pos) {
            const int nextPos = pos + 1;
            Forward(pos, nextPos);
            const bool generateToken = nextPos >= static_cast<int>(promptTokens.size());
            const int token = generateToken ? Sample(nextPos, generateToken) : promptTokens[nextPos];
            if (stopOnSpecial_ && token < 3)
                break;
            out.push_back(token);
        }
        return out;
    }

    std::vector<Half> Logits() const { return runstate->logits.ToHost(); }

    void Forward(int position, int nextPosition) // :158-190
    {
        if (decoder_) {
            Check(llama2_decode_forward(decoder_, position, nextPosition));
            return;
        }
        const int headSize = config.dim / config.n_heads;
        const float scale = 1.0f / std::sqrt(static_cast<float>(headSize));
        RunState& rs = *runstate;
        embedding.Forward(rs.x, weights->tokenEmbeddingTable, config.dim, rs.tokens, position);
        for (size_t i = 0; i < weights->layers.size(); ++i) {
            PerLayerWeight& layer = weights->layers[i];
            rmsNorm.Forward(rs.xb, rs.x, layer.rmsAttentionWeight, config.dim);
            const size_t layerOffset = i * static_cast<size_t>(config.seq_len) * kvDim;
            qkvMatVec.Forward(rs.q, rs.keyCache, rs.valueCache, rs.xb, layer.queryWeight, layer.keyWeight, layer.valueWeight,
                              config.dim, config.dim, layerOffset, position);
            rope.Forward(rs.q, rs.keyCache, config.n_kv_heads, headSize, position, layerOffset, config.rope_theta);
            MultiHeadAttention(rs.xb, rs.q, rs.keyCache, rs.valueCache, rs.attention, headSize, config.dim, nextPosition,
                               layerOffset, scale);
            matVecResidual.Forward(rs.x, rs.xb, layer.outputWeight, config.dim, config.dim);
            rmsNorm.Forward(rs.xb, rs.x, layer.rmsFeedForwardWeight, config.dim);
            matVecSwiGLU.Forward(rs.h, rs.xb, layer.gateWeight, layer.upWeight, config.dim, config.hidden_dim);
            matVecResidual.Forward(rs.x, rs.h, layer.downWeight, config.hidden_dim, config.dim);
        }
        rmsNorm.Forward(rs.x, rs.x, weights->rmsFinalWeight, config.dim);
        matVec.Forward(rs.logits, rs.x, weights->classifierWeights, config.dim, config.vocab_size);
    }

    Config config;
    int kvDim = 0;
    std::unique_ptr<TransformerWeights> weights;
    std::unique_ptr<RunState> runstate;

  private:
    int Sample(int nextPos, bool generateToken)
    {
        if (decoder_) {
            int token = 0;
            Check(llama2_decode_sample_top_p(decoder_, nextPos, generateToken ? 1 : 0, sampler->Temperature(),
                                             sampler->TopP(), sampler->Coin(nextPos), &token));
            return token;
        }
        return sampler->Sample(nextPos, generateToken);
    }
    void MultiHeadAttention(DeviceVariable<Half>& output, DeviceVariable<Half>& query, DeviceVariable<Half>& key,
                            DeviceVariable<Half>& value, DeviceVariable<Half>& attention, int headSize, int dim, int seqLength,
                            size_t layerOffset, float scale) // :150-156
    {
        matVecStrided.Forward(attention, query, key, headSize, dim, seqLength, layerOffset, scale);
        softmax.Forward(attention, seqLength);
        vecMat.Forward(output, value, attention, headSize, dim, seqLength, layerOffset);
    }

    std::unique_ptr<Sampler> sampler;
    Embedding embedding;
    RMSNorm rmsNorm;
    QKVMatVec qkvMatVec;
    RoPERotation rope;
    MatVecStrided matVecStrided;
    Softmax softmax;
    VecMat vecMat;
    MatVecResidual matVecResidual;
    MatVecSwiGLU matVecSwiGLU;
    MatVec matVec;
    std::vector<llama2_layer_weights> layerViews_;
    llama2_decoder* decoder_ = nullptr;
    bool stopOnSpecial_;
};

} // namespace libLlama2
