// C facade over the C++ host layer (llama2_host.hpp) so that the pytest suite
// can drive libLlama2::Transformer the way an application drives the
// reference's ITransformer.  Builds into libllama2_host.so.
#include "llama2_host.hpp"

#include <algorithm>
#include <string>

using namespace libLlama2;

namespace {
thread_local std::string g_error;

template <class F>
int guarded(F&& f)
{
    try {
        f();
        g_error.clear();
        return 0;
    } catch (const FileLoadException& e) {
        g_error = std::string("FileLoadException: ") + e.what();
        return 1;
    } catch (const NotImplementedException& e) {
        g_error = std::string("NotImplementedException: ") + e.what();
        return 2;
    } catch (const Llama2Exception& e) {
        g_error = std::string("Llama2Exception: ") + e.what();
        return 3;
    } catch (const std::exception& e) {
        g_error = std::string("exception: ") + e.what();
        return 4;
    }
}
} // namespace

extern "C" {

__attribute__((visibility("default"))) const char* l2h_last_error(void) { return g_error.c_str(); }

// The checks the Transformer constructor makes on a model file before it touches
// the GPU contents: header, GQA, size of the tensor stream.  No GPU needed.
__attribute__((visibility("default"))) int l2h_check_model_file(const char* path)
{
    return guarded([&] {
        MappedFile file(path);
        Config c = Config::LoadConfig(file.data(), file.size());
        if (c.kvDim() != c.dim)
            throw NotImplementedException("Differing kvDim dimention not currently supported.");
        const size_t remaining = file.size() - Config::Size;
        if (TransformerWeights::ExpectedBytes(c) != remaining)
            throw FileLoadException("Failed to read file. offset: " + std::to_string(TransformerWeights::ExpectedBytes(c)) +
                                    " != length: " + std::to_string(remaining));
    });
}

// ModelConverter::RepackQWeight on caller-provided host arrays; out_* sized as in the model file.
__attribute__((visibility("default"))) int l2h_repack_qweight(const uint32_t* qweight, const uint32_t* qzeros,
                                                              const uint16_t* scales, int height, int width, int format,
                                                              uint32_t* out_weight, uint32_t* out_zeros, uint16_t* out_scales)
{
    return guarded([&] {
        Check(llama2_init(0));
        auto r = ModelConverter::RepackQWeight(qweight, qzeros, scales, height, width,
                                               format == 0 ? ModelConverter::Format::v0 : ModelConverter::Format::v1);
        std::copy(r.Weight.begin(), r.Weight.end(), out_weight);
        std::copy(r.Zeros.begin(), r.Zeros.end(), out_zeros);
        std::copy(r.Scales.begin(), r.Scales.end(), out_scales);
    });
}

__attribute__((visibility("default"))) int l2h_transformer_open(const char* path, int mode, int stop_on_special, void** handle)
{
    *handle = nullptr;
    return guarded([&] { *handle = new Transformer(path, static_cast<Transformer::Mode>(mode), stop_on_special != 0); });
}

__attribute__((visibility("default"))) int l2h_transformer_open_sampled(const char* path, int mode, int stop_on_special,
                                                                        float temperature, float top_p,
                                                                        unsigned long long seed, void** handle)
{
    *handle = nullptr;
    return guarded([&] {
        *handle = new Transformer(path, static_cast<Transformer::Mode>(mode), stop_on_special != 0, temperature, top_p, seed);
    });
}

__attribute__((visibility("default"))) int l2h_transformer_generate(void* handle, const int* prompt, int n_prompt, int steps,
                                                                    int* out, int* n_out)
{
    return guarded([&] {
        auto* t = static_cast<Transformer*>(handle);
        std::vector<int> tokens = t->Generate(std::vector<int>(prompt, prompt + n_prompt), steps);
        for (size_t i = 0; i < tokens.size(); ++i)
            out[i] = tokens[i];
        *n_out = static_cast<int>(tokens.size());
    });
}

__attribute__((visibility("default"))) int l2h_transformer_logits(void* handle, uint16_t* out, int n)
{
    return guarded([&] {
        std::vector<Half> l = static_cast<Transformer*>(handle)->Logits();
        for (int i = 0; i < n && i < static_cast<int>(l.size()); ++i)
            out[i] = l[i];
    });
}

__attribute__((visibility("default"))) int l2h_transformer_seq_len(void* handle)
{
    return static_cast<Transformer*>(handle)->config.seq_len;
}

__attribute__((visibility("default"))) int l2h_transformer_close(void* handle)
{
    return guarded([&] { delete static_cast<Transformer*>(handle); });
}

} // extern "C"
